#include <memory>
#include "kernelmatrix.h"
#include <stdexcept>

#include <algorithm>
#include <cstdio>
#include <cstdlib>

using tsvm::abi_check;

namespace tsvm {
size_t &device_bytes_in_use() {
    static size_t bytes = 0;
    return bytes;
}

std::recursive_mutex &device_work_mutex() {
    static std::recursive_mutex m;
    return m;
}

RowArena &RowArena::instance() {
    static RowArena arena;
    return arena;
}

size_t RowArena::auto_budget() {
    if (full_budget_) return cap_;   // the arena already is the budget: never chase small changes in free memory
    size_t free_b = 0, total_b = 0;
    TSVM_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    // Nine tenths of what is free or already held, unless TSVM_ARENA_PERCENT (10..95) says otherwise: kernel rows
    // are what the memory is for (hits grow in proportion to the slots; the set-up of a class pair or a prediction
    // takes a few GB at most, and partial sums of predictions come out of the arena itself).  On the seven-class and
    // the regression benchmark: half 1.80 s / 1.77 s, three quarters 1.71 / 1.63, 85 % 1.68 / 1.59 with the kernels
    // of that time; with the present ones three quarters 1.576 / 1.586 (hits 46.8 % / 37.7 %), nine tenths
    // 1.530 / 1.550 (50.9 % / 43.7 %).
    const char *e = getenv("TSVM_ARENA_PERCENT");
    const int asked = e ? atoi(e) : 90;
    const size_t pct = (size_t) (asked < 10 ? 10 : asked > 95 ? 95 : asked);
    return (free_b + cap_) / 100 * pct;
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

// CSR assembly on the host (kernelmatrix.cpp:183-207): n_features = largest feature id + 1, ids kept
// as given; self dot products from the CSR values in stored order; then the layout is chosen.
std::shared_ptr<DeviceRows> DeviceRows::from_host(const DataSet::node2d &all, const int *rows, size_t n_rows) {
    auto out = std::make_shared<DeviceRows>();
    DeviceRows &r = *out;
    r.n = n_rows;
    std::vector<int64_t> ptr(n_rows + 1, 0);
    int max_index = 0;
#pragma omp parallel for reduction(max : max_index) schedule(static)
    for (size_t i = 0; i < n_rows; ++i) {
        const auto &row = all[rows ? rows[i] : i];
        ptr[i + 1] = (int64_t) row.size();
        for (const auto &nd : row) max_index = std::max(max_index, nd.index);
    }
    for (size_t i = 0; i < n_rows; ++i) ptr[i + 1] += ptr[i];
    r.nnz = (size_t) ptr[n_rows];
    r.n_features = (size_t) max_index + 1;
    // (not value-initialised: a std::vector would be zero-filled by one thread, 12 bytes per non-zero, before the
    // threads below write every element anyway)
    std::unique_ptr<kernel_type[]> val(new kernel_type[r.nnz]);
    std::unique_ptr<int[]> col(new int[r.nnz]);
    int all_float = 1;
#pragma omp parallel for schedule(static) reduction(min : all_float)
    for (size_t i = 0; i < n_rows; ++i) {
        const auto &row = all[rows ? rows[i] : i];
        size_t e = (size_t) ptr[i];
        for (const auto &nd : row) {
            val[e] = nd.value;
            col[e] = nd.index;
            if ((double) (float) nd.value != (double) nd.value) all_float = 0;
            ++e;
        }
    }
    r.values_fit_float = all_float != 0;
    r.val.resize(r.nnz);
    r.val.upload(val.get(), r.nnz);
    r.col.resize(r.nnz);
    r.col.upload(col.get(), r.nnz);
    r.row_ptr.upload(ptr);
    r.self_dot.resize(r.n);
    abi_check(tsvm_csr_self_dot(r.val.data(), r.row_ptr.data(), (int64_t) r.n, r.self_dot.data(), nullptr));
    r.dense = KernelMatrix::choose_dense(r.n, r.n_features, r.nnz);
    if (r.dense) {
        r.ld = (int64_t) ((r.n_features + 7) / 8 * 8);
        r.x.resize(r.n * (size_t) r.ld);
        abi_check(tsvm_csr_to_dense(r.val.data(), r.col.data(), r.row_ptr.data(), (int64_t) r.n, r.x.data(), r.ld, nullptr));
        TSVM_HIP_CHECK(hipDeviceSynchronize());
        r.val.release();
        r.col.release();
        r.row_ptr.release();
        r.find_indicator_columns();
    } else {
        r.host_row_ptr = std::move(ptr);
        r.build_sliced();
    }
    return out;
}

// The sliced copy of CSR rows (row offsets are known on the host).
void DeviceRows::build_sliced() {
    sliced_lds = 0;
    max_row_nnz = 0;
    if (dense || n == 0 || getenv("TSVM_NO_SLICED")) return;
    for (size_t i = 0; i < n; ++i) max_row_nnz = std::max(max_row_nnz, (int) (host_row_ptr[i + 1] - host_row_ptr[i]));
    const int vt = values_fit_float ? TSVM_ROW_F32 : TSVM_ROW_F64;
    const size_t need = tsvm_get_rows_csr_sliced_lds((int) n_features, max_row_nnz, vt);
    if (need == 0) return;
    const size_t n_slices = (n + 63) / 64;
    std::vector<int64_t> sp(n_slices + 1, 0);
    for (size_t s = 0; s < n_slices; ++s) {
        int64_t w = 0;
        for (size_t i = s * 64; i < std::min(n, s * 64 + 64); ++i) w = std::max(w, host_row_ptr[i + 1] - host_row_ptr[i]);
        sp[s + 1] = sp[s] + 64 * w;
    }
    // (a few very long rows would blow the padded copy up: then the plain CSR kernel stays in charge)
    if ((size_t) sp[n_slices] > 4 * nnz + 64 * n_slices) return;
    if (sp[n_slices] == 0) return;   // every row is empty: nothing to slice, the plain kernel writes kappa(0, 0)
    slice_ptr.upload(sp);
    ell_col.resize((size_t) sp[n_slices]);
    ell_val.resize((size_t) sp[n_slices] * (values_fit_float ? sizeof(float) : sizeof(double)));
    abi_check(tsvm_csr_to_sliced(val.data(), col.data(), row_ptr.data(), (int64_t) n, slice_ptr.data(), (int) n_features, ell_col.data(),
                                 ell_val.data(), vt, nullptr));
    TSVM_HIP_CHECK(hipDeviceSynchronize());
    sliced_lds = need;
}

std::shared_ptr<DeviceRows> DeviceRows::subset(const DeviceRows &base, const int *rows, size_t n_rows) {
    auto out = std::make_shared<DeviceRows>();
    DeviceRows &r = *out;
    r.n = n_rows;
    r.n_features = base.n_features;
    r.dense = base.dense;
    r.values_fit_float = base.values_fit_float;
    r.ld = base.ld;
    tsvm::DeviceBuffer<int> d_rows(n_rows);
    d_rows.upload(rows, n_rows);
    r.self_dot.resize(n_rows);
    abi_check(tsvm_gather_f64(base.self_dot.data(), d_rows.data(), (int) n_rows, r.self_dot.data(), nullptr));
    if (base.dense) {
        r.x.resize(n_rows * (size_t) r.ld);
        abi_check(tsvm_gather_rows_f64(base.x.data(), base.ld, d_rows.data(), (int64_t) n_rows, r.x.data(), nullptr));
        r.nnz = n_rows ? base.nnz / std::max<size_t>(base.n, 1) * n_rows : 0;   // estimate, informational only
        if (base.ind_first >= 0) {   // indicator columns of all rows are indicator columns of a subset (masks move as 8-byte words)
            r.ind_first = base.ind_first;
            r.ind_max_ones = base.ind_max_ones;
            r.ind_mask.resize(n_rows);
            abi_check(tsvm_gather_f64(reinterpret_cast<const double *>(base.ind_mask.data()), d_rows.data(), (int) n_rows,
                                      reinterpret_cast<double *>(r.ind_mask.data()), nullptr));
        }
    } else {
        r.host_row_ptr.assign(n_rows + 1, 0);
        for (size_t i = 0; i < n_rows; ++i)
            r.host_row_ptr[i + 1] = r.host_row_ptr[i] + base.host_row_ptr[rows[i] + 1] - base.host_row_ptr[rows[i]];
        r.nnz = (size_t) r.host_row_ptr[n_rows];
        r.row_ptr.upload(r.host_row_ptr);
        r.val.resize(r.nnz);
        r.col.resize(r.nnz);
        abi_check(tsvm_csr_gather_rows(base.val.data(), base.col.data(), base.row_ptr.data(), d_rows.data(), (int64_t) n_rows,
                                       r.row_ptr.data(), r.val.data(), r.col.data(), nullptr));
        r.build_sliced();
    }
    TSVM_HIP_CHECK(hipDeviceSynchronize());   // d_rows is released on return
    return out;
}

const std::vector<int> &DeviceRows::column_stats() const {
    if (column_stats_.size() != 2 * n_features) {
        tsvm::DeviceBuffer<int> d_counts(2 * n_features);
        if (dense) abi_check(tsvm_column_stats_dense(x.data(), ld, (int64_t) n, (int) n_features, d_counts.data(), nullptr));
        else abi_check(tsvm_column_stats_csr(val.data(), col.data(), (int64_t) nnz, (int) n_features, d_counts.data(), nullptr));
        column_stats_ = d_counts.to_host();
    }
    return column_stats_;
}

// The trailing run of columns whose values are all 0 or 1 (at most 64 of them): its first column, n_features when
// the last column is not such a column.  stats: the 2 * n_features counts of column_stats().
int DeviceRows::indicator_run_start(const int *stats, int n_features) {
    int first = n_features;
    while (first > 0 && n_features - first < 64 && stats[n_features + first - 1] == 0) --first;
    return first;
}

// Leaving the run to the kernel's epilogue pays when it saves more than the additions cost there: one 4-column step
// of the matrix cores per value is worth about one epilogue instruction, an indicator column that may match about three.
bool DeviceRows::indicator_run_pays(int n_features, int first, int max_ones) {
    const int steps_saved = (n_features + 3) / 4 - (first + 3) / 4;
    return steps_saved >= 2 + 3 * max_ones;
}

void DeviceRows::find_indicator_columns() {
    ind_first = -1;
    if (!dense || n == 0 || n_features == 0 || getenv("TSVM_NO_INDICATOR")) return;
    const std::vector<int> &stats = column_stats();
    const int first = indicator_run_start(stats.data(), (int) n_features);
    if (first == (int) n_features) return;
    tsvm::DeviceBuffer<uint64_t> masks(n);
    tsvm::DeviceBuffer<int> d_max(1);
    abi_check(tsvm_indicator_masks(x.data(), ld, (int64_t) n, first, (int) n_features - first, masks.data(), d_max.data(), nullptr));
    const int max_ones = d_max.to_host()[0];
    if (!indicator_run_pays((int) n_features, first, max_ones)) return;
    ind_first = first;
    ind_max_ones = max_ones;
    ind_mask = std::move(masks);
}

std::shared_ptr<DeviceRows> DeviceRows::of(const DataSet &dataset) {
    std::shared_ptr<void> &slot = dataset.device_cache();
    if (!slot) slot = from_host(dataset.instances(), nullptr, dataset.instances().size());
    return std::static_pointer_cast<DeviceRows>(slot);
}

KernelMatrix::KernelMatrix(const DataSet::node2d &instances, SvmParam param) : param(param) {
    rows_ = DeviceRows::from_host(instances, nullptr, instances.size());
    finish(1);
}

KernelMatrix::KernelMatrix(const DataSet::node2d &all, const int *rows, size_t n_rows, SvmParam param, int repeat)
    : param(param) {
    rows_ = DeviceRows::from_host(all, rows, n_rows);
    finish(repeat);
}

KernelMatrix::KernelMatrix(const DataSet &dataset, const int *rows, size_t n_rows, SvmParam param, int repeat)
    : param(param) {
    std::shared_ptr<DeviceRows> all = DeviceRows::of(dataset);
    rows_ = rows ? DeviceRows::subset(*all, rows, n_rows) : all;
    finish(repeat);
}

// diag from the self dot products (kernelmatrix.cpp:225-247).  With repeat > 1 the reference stacks the
// same rows several times (the 2n-row problem of SVR, svr.cpp:14-15); here the rows are stored once and
// only the diagonal, which the solver kernels index by instance id, is replicated.
void KernelMatrix::finish(int repeat) {
    n_unique_ = rows_->n;
    repeat_ = repeat;
    diag_.resize(n_unique_ * repeat_);
    abi_check(tsvm_kernel_diag(rows_->self_dot.data(), (int64_t) n_unique_, (int) param.kernel_type, param.gamma, param.coef0,
                               param.degree, diag_.data(), nullptr));
    for (int rep = 1; rep < repeat_; ++rep)
        TSVM_HIP_CHECK(hipMemcpyAsync(diag_.data() + rep * n_unique_, diag_.data(), n_unique_ * sizeof(kernel_type),
                                      hipMemcpyDeviceToDevice, nullptr));
    TSVM_HIP_CHECK(hipDeviceSynchronize());
}

size_t KernelMatrix::reference_syncmem_bytes() const {
    const DeviceRows &R = *rows_;
    const std::vector<int> &stats = R.column_stats();
    const long long nf = (long long) R.n_features, m = (long long) n_instances();
    std::vector<long long> cnt(nf);
    long long entries = 0;
    for (long long c = 0; c < nf; ++c) {
        cnt[c] = (long long) stats[c] * repeat_;
        entries += cnt[c];
    }
    // columns by entry count ascending, ties by index (kernelmatrix.cpp:32-41); leading columns go to the sparse part
    // while the part stays under 5 % full, the column under 50 % full, and four times its entries do not exceed
    // the cells left to the dense part (kernelmatrix.cpp:58-74)
    std::vector<int> order(nf);
    for (long long c = 0; c < nf; ++c) order[c] = (int) c;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return cnt[a] != cnt[b] ? cnt[a] < cnt[b] : a < b; });
    long long total_csr = 0, total_dense = m * nf, row_sum = 0, dense_cols = nf, nnz_sparse = 0;
    for (long long i = 0; i < nf; ++i) {
        const long long c = cnt[order[i]];
        total_csr += c;
        total_dense -= m;
        row_sum += m;
        if ((long double) total_csr / row_sum > 0.05 || (long double) c / m > 0.5 || total_csr * 4 > total_dense) break;
        --dense_cols;
        nnz_sparse += c;
    }
    size_t bytes = (size_t) entries * (sizeof(kernel_type) + sizeof(int)) + (size_t) (m + 1) * sizeof(int) +
                   2 * (size_t) m * sizeof(kernel_type);
    if (dense_cols > 0) bytes += (size_t) m * dense_cols * sizeof(kernel_type);                      // dense.val, kernelmatrix.cpp:79-83
    if (dense_cols < nf && nnz_sparse != 0)   // some entry lies outside the dense part (kernelmatrix.cpp:151-176)
        bytes += (size_t) nnz_sparse * (sizeof(kernel_type) + sizeof(int)) + (size_t) (m + 1) * sizeof(int);
    return bytes;
}

// A staging buffer that is all-zero whenever it is not in use: grown (and cleared) only when a call needs more.
static void grow_zeroed(tsvm::DeviceBuffer<unsigned char> &b, size_t bytes, hipStream_t stream) {
    if (b.size() >= bytes) return;
    b.resize(bytes);
    TSVM_HIP_CHECK(hipMemsetAsync(b.data(), 0, bytes, stream));
}

void KernelMatrix::get_rows(const int *d_idx, int m, void *d_out, int64_t ld, const int *d_out_slots,
                            hipStream_t stream) const {
    const DeviceRows &R = *rows_;
    const int n = (int) n_unique_;
    if (R.dense && R.ind_first >= 0) {
        abi_check(tsvm_get_rows_dense_indicator(R.x.data(), R.ld, nullptr, n, R.ind_first, R.self_dot.data(), R.ind_mask.data(),
                                                R.x.data(), R.ld, d_idx, m, nullptr, R.self_dot.data(), R.ind_mask.data(),
                                                R.ind_max_ones, (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                                d_out, row_type(), d_out_slots, ld, stream));
        return;
    }
    if (R.dense) {
        abi_check(tsvm_get_rows_dense(R.x.data(), R.ld, nullptr, n, (int) R.n_features, R.self_dot.data(), R.x.data(), R.ld, d_idx,
                                      m, R.self_dot.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, row_type(), d_out_slots, ld, stream));
        return;
    }
    const int wt = R.values_fit_float ? TSVM_ROW_F32 : TSVM_ROW_F64;
    if (R.sliced_lds) {   // the stored rows streamed once per sixteen working rows, the working rows in LDS
        abi_check(tsvm_get_rows_csr_sliced(R.ell_col.data(), R.ell_val.data(), wt, R.slice_ptr.data(), n, R.self_dot.data(),
                                           R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, R.self_dot.data(),
                                           (int) R.n_features, R.max_row_nnz, (int) param.kernel_type, param.gamma, param.coef0,
                                           param.degree, d_out, row_type(), d_out_slots, ld, stream));
        return;
    }
    // The staging matrix [n_features][m] is kept all-zero between uses: the working rows' non-zeros are written
    // into it and taken out again afterwards (nnz entries each way instead of a fill of n_features x m).
    grow_zeroed(stage_w_, (size_t) m * R.n_features * (R.values_fit_float ? sizeof(float) : sizeof(double)), stream);
    if (stage_sd_.size() < (size_t) m) stage_sd_.resize(m);
    abi_check(tsvm_csr_scatter_rows(R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, (int) R.n_features,
                                    stage_w_.data(), wt, 0, stream));
    abi_check(tsvm_gather_f64(R.self_dot.data(), d_idx, m, stage_sd_.data(), stream));
    abi_check(tsvm_get_rows_csr_staged(R.val.data(), R.col.data(), R.row_ptr.data(), nullptr, n, R.self_dot.data(),
                                       stage_w_.data(), wt, m, stage_sd_.data(), (int) param.kernel_type, param.gamma,
                                       param.coef0, param.degree, d_out, row_type(), d_out_slots, ld, stream));
    abi_check(tsvm_csr_scatter_rows(R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, (int) R.n_features,
                                    stage_w_.data(), wt, 1, stream));
}

void KernelMatrix::get_rows_counted(const int *d_idx, int m_max, const int *d_m, void *d_out, int64_t ld,
                                    const int *d_out_slots, hipStream_t stream) const {
    const DeviceRows &R = *rows_;
    if (!R.dense) throw std::logic_error("KernelMatrix::get_rows_counted: dense layout only");
    if (R.ind_first >= 0) {
        abi_check(tsvm_get_rows_dense_indicator(R.x.data(), R.ld, nullptr, (int) n_unique_, R.ind_first, R.self_dot.data(),
                                                R.ind_mask.data(), R.x.data(), R.ld, d_idx, m_max, d_m, R.self_dot.data(),
                                                R.ind_mask.data(), R.ind_max_ones, (int) param.kernel_type, param.gamma,
                                                param.coef0, param.degree, d_out, row_type(), d_out_slots, ld, stream));
        return;
    }
    abi_check(tsvm_get_rows_dense_counted(R.x.data(), R.ld, nullptr, (int) n_unique_, (int) R.n_features, R.self_dot.data(),
                                          R.x.data(), R.ld, d_idx, m_max, d_m, R.self_dot.data(), (int) param.kernel_type,
                                          param.gamma, param.coef0, param.degree, d_out, row_type(), d_out_slots, ld, stream));
}

// K(x_idx[r], x_idx[t]) for r, t < m: the same kernels with the column set restricted to the m rows,
// so every value is bit-identical to the corresponding entry of a full kernel row.  Elements are row_type() wide.
void KernelMatrix::get_block(const int *d_idx, int m, void *d_out, int64_t ld, hipStream_t stream) const {
    const DeviceRows &R = *rows_;
    if (R.dense) {
        abi_check(tsvm_get_rows_dense(R.x.data(), R.ld, d_idx, m, (int) R.n_features, R.self_dot.data(), R.x.data(), R.ld, d_idx, m,
                                      R.self_dot.data(), (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, row_type(), nullptr, ld, stream));
        return;
    }
    const int wt = R.values_fit_float ? TSVM_ROW_F32 : TSVM_ROW_F64;
    // kept all-zero between uses, as in get_rows
    grow_zeroed(stage_blk_, (size_t) m * R.n_features * (R.values_fit_float ? sizeof(float) : sizeof(double)), stream);
    if (stage_blk_sd_.size() < (size_t) m) stage_blk_sd_.resize(m);
    abi_check(tsvm_csr_scatter_rows(R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, (int) R.n_features,
                                    stage_blk_.data(), wt, 0, stream));
    abi_check(tsvm_gather_f64(R.self_dot.data(), d_idx, m, stage_blk_sd_.data(), stream));
    abi_check(tsvm_get_rows_csr_staged(R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, R.self_dot.data(),
                                       stage_blk_.data(), wt, m, stage_blk_sd_.data(), (int) param.kernel_type, param.gamma,
                                       param.coef0, param.degree, d_out, row_type(), nullptr, ld, stream));
    abi_check(tsvm_csr_scatter_rows(R.val.data(), R.col.data(), R.row_ptr.data(), d_idx, m, (int) R.n_features,
                                    stage_blk_.data(), wt, 1, stream));
}

// External batch (kernelmatrix.cpp:281-312, 385-406): features with id >= R.n_features are left out of
// the dot product but stay in the batch row's self dot.
void KernelMatrix::get_rows(const DataSet::node2d &instances, void *d_out, int64_t ld) const {
    get_rows(instances.data(), instances.size(), d_out, ld);
}

// The batch goes to the device as CSR (flattened by all cores into pinned memory, copied asynchronously) together
// with its rows' self dot products; with dense stored rows it is also laid out as a dense matrix of the stored rows'
// width (columns >= n_features are dropped from the products, kernelmatrix.cpp:392, but stay in the self dot).
KernelMatrix::StagedBatch KernelMatrix::stage_batch(const std::vector<DataSet::node> *instances, size_t n_rows) const {
    const DeviceRows &R = *rows_;
    const int m = (int) n_rows;
    TSVM_HIP_CHECK(hipStreamSynchronize(nullptr));   // a previous batch's copies have left the staging memory
    h_ptr_.reserve((size_t) m + 1);
    int64_t *ptr = h_ptr_.data();
    ptr[0] = 0;
    for (int r = 0; r < m; ++r) ptr[r + 1] = ptr[r] + (int64_t) instances[r].size();
    const size_t total = (size_t) ptr[m];
    h_val_.reserve(total);
    h_col_.reserve(total);
    kernel_type *val = h_val_.data();
    int *col = h_col_.data();
    // (indicator columns of the stored rows: the batch can use them when its own values there are zeros and ones)
    const int ind_lo = R.ind_first >= 0 ? R.ind_first : 0x7fffffff, ind_hi = (int) R.n_features;
    int not_indicator = 0;
#pragma omp parallel for schedule(static) reduction(max : not_indicator)
    for (int r = 0; r < m; ++r) {
        size_t e = (size_t) ptr[r];
        for (const auto &nd : instances[r]) {
            val[e] = nd.value;
            col[e] = nd.index;
            if (nd.index >= ind_lo && nd.index < ind_hi && nd.value != 0.0 && nd.value != 1.0) not_indicator = 1;
            ++e;
        }
    }
    if (b_val_.size() < total) { b_val_.resize(total); b_col_.resize(total); }
    if (b_ptr_.size() < (size_t) m + 1) b_ptr_.resize(m + 1);
    if (total) {
        TSVM_HIP_CHECK(hipMemcpyAsync(b_val_.data(), val, total * sizeof(kernel_type), hipMemcpyHostToDevice, nullptr));
        TSVM_HIP_CHECK(hipMemcpyAsync(b_col_.data(), col, total * sizeof(int), hipMemcpyHostToDevice, nullptr));
    }
    TSVM_HIP_CHECK(hipMemcpyAsync(b_ptr_.data(), ptr, ((size_t) m + 1) * sizeof(int64_t), hipMemcpyHostToDevice, nullptr));
    if (stage_sd_.size() < (size_t) m) stage_sd_.resize(m);
    abi_check(tsvm_csr_self_dot(b_val_.data(), b_ptr_.data(), m, stage_sd_.data(), nullptr));
    StagedBatch out;
    out.sd = stage_sd_.data();
    out.indicator_values = R.ind_first >= 0 && !not_indicator;
    if (R.dense) {
        if (stage_.size() < (size_t) m * R.ld) stage_.resize((size_t) m * R.ld);
        abi_check(tsvm_csr_to_dense(b_val_.data(), b_col_.data(), b_ptr_.data(), m, stage_.data(), R.ld, nullptr));
        out.a = stage_.data();
        out.lda = R.ld;
    }
    return out;
}

void KernelMatrix::get_rows(const std::vector<DataSet::node> *instances, size_t n_rows, void *d_out, int64_t ld) const {
    const DeviceRows &R = *rows_;
    const int m = (int) n_rows;
    if (m == 0) return;
    const StagedBatch b = stage_batch(instances, n_rows);
    const int n = (int) n_unique_;
    if (R.dense) {
        abi_check(tsvm_get_rows_dense(R.x.data(), R.ld, nullptr, n, (int) R.n_features, R.self_dot.data(), b.a, b.lda, nullptr, m,
                                      b.sd, (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                      d_out, row_type(), nullptr, ld, nullptr));
    } else {
        if (stage_.size() < (size_t) m * R.n_features) stage_.resize((size_t) m * R.n_features);
        abi_check(tsvm_csr_stage_rows(b_val_.data(), b_col_.data(), b_ptr_.data(), nullptr, m, (int) R.n_features,
                                      stage_.data(), nullptr));
        abi_check(tsvm_get_rows_csr(R.val.data(), R.col.data(), R.row_ptr.data(), nullptr, n, R.self_dot.data(), stage_.data(), m,
                                    b.sd, (int) param.kernel_type, param.gamma, param.coef0, param.degree,
                                    d_out, row_type(), nullptr, ld, nullptr));
    }
}
