#include "kernelmatrix.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

using tsvm::abi_check;

namespace tsvm {
size_t &device_bytes_in_use() {
    static size_t bytes = 0;
    return bytes;
}

RowArena &RowArena::instance() {
    static RowArena arena;
    return arena;
}

size_t RowArena::auto_budget() {
    if (full_budget_) return cap_;   // the arena already is the budget: never chase small changes in free memory
    size_t free_b = 0, total_b = 0;
    TSVM_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    return (free_b + cap_) / 2;   // what the arena already holds counts as available to it
}

// The arena only ever grows.  Small requests (tests, small problems) get twice what they ask for, so
// that little is held and little has to be scrubbed by the driver when the process ends (giving back
// ~140 GB was measured to stall the next process on the device for 2-3 s).  A request above a quarter
// of the automatic budget takes the whole budget at once: a multi-class run then allocates a single
// time instead of releasing and re-allocating tens of gigabytes between its sub-problems, each release
// costing up to a second.
void *RowArena::acquire(size_t bytes, bool auto_sized) {
    if (bytes <= cap_) return ptr_;
    size_t want = bytes;
    bool take_all = false;
    if (auto_sized) {
        const size_t budget = auto_budget();
        take_all = bytes > budget / 4;
        want = take_all ? std::max(bytes, budget) : std::max(bytes * 2, cap_ + cap_ / 2);
    }
    release();
    TSVM_HIP_CHECK(hipMalloc(&ptr_, want));
    cap_ = want;
    full_budget_ = take_all;
    static bool registered = false;
    if (!registered) {
        registered = true;
        atexit([] { RowArena::instance().release(); });
    }
    return ptr_;
}

void RowArena::release() {
    if (ptr_) (void) hipFree(ptr_);
    ptr_ = nullptr;
    cap_ = 0;
    full_budget_ = false;
}
}  // namespace tsvm

// Dense rows cost d_pad MFMA k-steps per output, CSR rows cost one L2 gather per stored non-zero;
// the matrix cores run roughly 30 k-steps in the time of one gather, so dense wins unless rows
// are very sparse.  Dense storage is also capped at 64 GiB.
bool KernelMatrix::choose_dense(size_t n, size_t n_features, size_t nnz) {
    if (n == 0) return true;
    const size_t ld = (n_features + 7) / 8 * 8;
    const double avg = (double) nnz / (double) n;
    if ((double) ld * (double) n * 8.0 > 64.0 * 1024 * 1024 * 1024) return false;
    return (double) ld <= 32.0 * std::max(avg, 1.0);
}

KernelMatrix::KernelMatrix(const DataSet::node2d &instances, SvmParam param) : param(param) {
    build(instances, nullptr, instances.size(), 1);
}

KernelMatrix::KernelMatrix(const DataSet::node2d &all, const int *rows, size_t n_rows, SvmParam param, int repeat)
    : param(param) {
    build(all, rows, n_rows, repeat);
}

// CSR assembly on the host (kernelmatrix.cpp:183-207): n_features_ = largest feature id + 1, ids kept
// as given.  With repeat > 1 the reference stacks the same rows several times (the 2n-row problem of
// SVR, svr.cpp:14-15); here the rows are stored once.
void KernelMatrix::build(const DataSet::node2d &all, const int *rows, size_t n_rows, int repeat) {
    n_unique_ = n_rows;
    repeat_ = repeat;
    std::vector<int64_t> ptr(n_rows + 1, 0);
    int max_index = 0;
#pragma omp parallel for reduction(max : max_index) schedule(static)
    for (size_t r = 0; r < n_rows; ++r) {
        const auto &row = all[rows ? rows[r] : r];
        ptr[r + 1] = (int64_t) row.size();
        for (const auto &nd : row) max_index = std::max(max_index, nd.index);
    }
    for (size_t r = 0; r < n_rows; ++r) ptr[r + 1] += ptr[r];
    nnz_ = (size_t) ptr[n_rows];
    n_features_ = (size_t) max_index + 1;
    std::vector<kernel_type> val(nnz_);
    std::vector<int> col(nnz_);
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < n_rows; ++r) {
        const auto &row = all[rows ? rows[r] : r];
        size_t e = (size_t) ptr[r];
        for (const auto &nd : row) { val[e] = nd.value; col[e] = nd.index; ++e; }
    }
    val_.upload(val);
    col_ind_.upload(col);
    row_ptr_.upload(ptr);
    self_dot_.resize(n_unique_);
    diag_.resize(n_unique_ * repeat_);
    abi_check(tsvm_csr_self_dot(val_.data(), row_ptr_.data(), (int64_t) n_unique_, self_dot_.data(), nullptr));
    abi_check(tsvm_kernel_diag(self_dot_.data(), (int64_t) n_unique_, (int) param.kernel_type, param.gamma, param.coef0,
                               param.degree, diag_.data(), nullptr));
    for (int rep = 1; rep < repeat_; ++rep)
        TSVM_HIP_CHECK(hipMemcpyAsync(diag_.data() + rep * n_unique_, diag_.data(), n_unique_ * sizeof(kernel_type),
                                      hipMemcpyDeviceToDevice, nullptr));
    dense_ = choose_dense(n_unique_, n_features_, nnz_);
    if (dense_) {
        ld_ = (int64_t) ((n_features_ + 7) / 8 * 8);
        x_.resize(n_unique_ * (size_t) ld_);
        abi_check(tsvm_csr_to_dense(val_.data(), col_ind_.data(), row_ptr_.data(), (int64_t) n_unique_, x_.data(), ld_,
                                    nullptr));
        TSVM_HIP_CHECK(hipDeviceSynchronize());
        val_.release();
        col_ind_.release();
        row_ptr_.release();
    }
}

void KernelMatrix::get_rows(const int *d_idx, int m, void *d_out, int64_t ld, const int *d_out_slots,
                            hipStream_t stream) const {
    const int n = (int) n_unique_;
    if (dense_) {
        abi_check(tsvm_get_rows_dense(x_.data(), ld_, nullptr, n, (int) n_features_, self_dot_.data(), x_.data(), ld_, d_idx,
                                      m, self_dot_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, row_type(), d_out_slots, ld, stream));
        return;
    }
    if (stage_.size() < (size_t) m * n_features_) stage_.resize((size_t) m * n_features_);
    if (stage_sd_.size() < (size_t) m) stage_sd_.resize(m);
    abi_check(tsvm_csr_stage_rows(val_.data(), col_ind_.data(), row_ptr_.data(), d_idx, m, (int) n_features_,
                                  stage_.data(), stream));
    abi_check(tsvm_gather_f64(self_dot_.data(), d_idx, m, stage_sd_.data(), stream));
    abi_check(tsvm_get_rows_csr(val_.data(), col_ind_.data(), row_ptr_.data(), nullptr, n, self_dot_.data(), stage_.data(),
                                m, stage_sd_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree, d_out,
                                row_type(), d_out_slots, ld, stream));
}

// K(x_idx[r], x_idx[t]) for r, t < m: the same kernels with the column set restricted to the m rows,
// so every value is bit-identical to the corresponding entry of a full kernel row.
void KernelMatrix::get_block(const int *d_idx, int m, kernel_type *d_out, int64_t ld, hipStream_t stream) const {
    if (dense_) {
        abi_check(tsvm_get_rows_dense(x_.data(), ld_, d_idx, m, (int) n_features_, self_dot_.data(), x_.data(), ld_, d_idx, m,
                                      self_dot_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, TSVM_ROW_F64, nullptr, ld, stream));
        return;
    }
    if (stage_blk_.size() < (size_t) m * n_features_) stage_blk_.resize((size_t) m * n_features_);
    if (stage_blk_sd_.size() < (size_t) m) stage_blk_sd_.resize(m);
    abi_check(tsvm_csr_stage_rows(val_.data(), col_ind_.data(), row_ptr_.data(), d_idx, m, (int) n_features_,
                                  stage_blk_.data(), stream));
    abi_check(tsvm_gather_f64(self_dot_.data(), d_idx, m, stage_blk_sd_.data(), stream));
    abi_check(tsvm_get_rows_csr(val_.data(), col_ind_.data(), row_ptr_.data(), d_idx, m, self_dot_.data(), stage_blk_.data(),
                                m, stage_blk_sd_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                d_out, TSVM_ROW_F64, nullptr, ld, stream));
}

// External batch (kernelmatrix.cpp:281-312, 385-406): features with id >= n_features_ are left out of
// the dot product but stay in the batch row's self dot.
void KernelMatrix::get_rows(const DataSet::node2d &instances, void *d_out, int64_t ld) const {
    const int m = (int) instances.size();
    if (m == 0) return;
    std::vector<int64_t> ptr(m + 1, 0);
    size_t total = 0;
    for (const auto &row : instances) total += row.size();
    std::vector<kernel_type> val(total);
    std::vector<int> col(total);
    size_t e = 0;
    for (int r = 0; r < m; ++r) {
        for (const auto &nd : instances[r]) { val[e] = nd.value; col[e] = nd.index; ++e; }
        ptr[r + 1] = (int64_t) e;
    }
    if (b_val_.size() < total) { b_val_.resize(total); b_col_.resize(total); }
    if (b_ptr_.size() < (size_t) m + 1) b_ptr_.resize(m + 1);
    b_val_.upload(val.data(), total);
    b_col_.upload(col.data(), total);
    b_ptr_.upload(ptr.data(), m + 1);
    if (stage_sd_.size() < (size_t) m) stage_sd_.resize(m);
    abi_check(tsvm_csr_self_dot(b_val_.data(), b_ptr_.data(), m, stage_sd_.data(), nullptr));
    const int n = (int) n_unique_;
    if (dense_) {
        if (stage_.size() < (size_t) m * ld_) stage_.resize((size_t) m * ld_);
        // columns >= n_features_ are dropped: the staging matrix is only n_features_ wide
        abi_check(tsvm_csr_to_dense(b_val_.data(), b_col_.data(), b_ptr_.data(), m, stage_.data(), ld_, nullptr));
        abi_check(tsvm_get_rows_dense(x_.data(), ld_, nullptr, n, (int) n_features_, self_dot_.data(), stage_.data(), ld_, nullptr, m,
                                      stage_sd_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, row_type(), nullptr, ld, nullptr));
    } else {
        if (stage_.size() < (size_t) m * n_features_) stage_.resize((size_t) m * n_features_);
        abi_check(tsvm_csr_stage_rows(b_val_.data(), b_col_.data(), b_ptr_.data(), nullptr, m, (int) n_features_,
                                      stage_.data(), nullptr));
        abi_check(tsvm_get_rows_csr(val_.data(), col_ind_.data(), row_ptr_.data(), nullptr, n, self_dot_.data(), stage_.data(), m,
                                    stage_sd_.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                    d_out, row_type(), nullptr, ld, nullptr));
    }
}
