"""Two rules of the C++ host layer restated for callers that drive the kernel-level C ABI themselves (the benchmark's
kernel timings) and want the kernels a training run would use:

* choose_dense: KernelMatrix::choose_dense (thundersvm_amd/host/kernelmatrix.cpp): dense row-major storage unless the
  rows are very sparse or the dense copy would exceed 64 GiB;
* indicator_columns: DeviceRows::find_indicator_columns: the first column of the trailing run (at most 64 columns)
  whose values are all 0 or 1, from the counts of tsvm_column_stats_dense.
"""


def choose_dense(n, n_features, nnz):
    if n == 0:
        return True
    ld = (n_features + 7) // 8 * 8
    if float(ld) * n * 8.0 > 64.0 * 1024 ** 3:
        return False
    return ld <= 32.0 * max(nnz / n, 1.0)


def indicator_columns(counts, n_features):
    """counts: the 2 * n_features ints of tsvm_column_stats_dense.  Returns the first indicator column
    (n_features when there is no trailing indicator run)."""
    first = n_features
    while first > 0 and n_features - first < 64 and counts[n_features + first - 1] == 0:
        first -= 1
    return first
