// KernelMatrix: the training (or support-vector) rows resident in HBM, serving kernel rows by id or
// for an external batch.  Public surface of include/thundersvm/kernelmatrix.h:39-72 with device
// pointers in place of SyncArray.
//
// Layout in HBM: either dense row-major fp64 [n][ld] (ld = n_features rounded up to 8, column c =
// feature id c) for the MFMA path, or CSR (fp64 values, int32 columns, int64 row offsets) for the
// sparse path.  The layout is chosen from the average row fill (see choose_dense()).
//
// A matrix built with repeat = r stands for the reference's r*n-row matrix made of the same n rows
// stacked r times (SVR, svr.cpp:14-15).  Instance id i and i + n then have the same kernel row, and
// that row consists of r identical n-column pieces: only the n unique rows are stored, and kernel
// rows are produced under the folded id i % n, n columns wide.
//
// Kernel rows are produced as float for the RBF, polynomial and sigmoid kernels, whose values are
// float-rounded by definition, and as double for the linear kernel (row_type()).
#pragma once
#include "dataset.h"
#include "device.h"
#include "svmparam.h"

// A set of data rows resident in HBM (either layout) with their self dot products; what a KernelMatrix
// multiplies against.  A DataSet keeps one for all of its instances (DeviceRows::of), so that the
// one-vs-one sub-problems of a multi-class run take their rows from HBM with a device-side gather
// instead of being assembled on the host and uploaded once per class pair.
struct DeviceRows {
    size_t n = 0, n_features = 0, nnz = 0;
    bool dense = false;
    bool values_fit_float = false;               // every stored value is exactly a float (CSR layout: staging type)
    int64_t ld = 0;                              // dense row stride (n_features rounded up to 8)
    tsvm::DeviceBuffer<kernel_type> x;           // dense layout [n][ld]
    tsvm::DeviceBuffer<kernel_type> val;         // CSR layout
    tsvm::DeviceBuffer<int> col;
    tsvm::DeviceBuffer<int64_t> row_ptr;
    std::vector<int64_t> host_row_ptr;           // CSR layout only: needed to lay out a subset
    // CSR layout: the rows a second time in slices of 64 (sliced ELL, see tsvm_get_rows_csr_sliced), which get_rows
    // streams; values as float when values_fit_float.  sliced_lds == 0: the shape does not fit that kernel.
    tsvm::DeviceBuffer<int> ell_col;
    tsvm::DeviceBuffer<unsigned char> ell_val;
    tsvm::DeviceBuffer<int64_t> slice_ptr;
    int max_row_nnz = 0;
    size_t sliced_lds = 0;
    void build_sliced();
    tsvm::DeviceBuffer<kernel_type> self_dot;    // [n]
    // per column c < n_features: [c] = entries (dense: non-zero values; CSR: stored entries), [n_features + c] = values
    // that are neither 0 nor 1; counted on the device on first use
    const std::vector<int> &column_stats() const;
    mutable std::vector<int> column_stats_;
    // Dense layout: when the last columns hold only zeros and ones (one-hot encoded categories), columns
    // ind_first .. n_features-1 (at most 64) are also kept as one bit mask per row, and get_rows leaves them to the
    // kernel's epilogue instead of the matrix cores.  ind_first < 0: no such part.
    int ind_first = -1, ind_max_ones = 0;
    tsvm::DeviceBuffer<uint64_t> ind_mask;       // [n]
    void find_indicator_columns();
    static int indicator_run_start(const int *stats, int n_features);
    static bool indicator_run_pays(int n_features, int first, int max_ones);

    // rows[0..n_rows) of `all` (rows == nullptr: the first n_rows), assembled on the host and uploaded
    static std::shared_ptr<DeviceRows> from_host(const DataSet::node2d &all, const int *rows, size_t n_rows);
    // rows[0..n_rows) of `base`, gathered on the device; keeps base's layout and feature count
    static std::shared_ptr<DeviceRows> subset(const DeviceRows &base, const int *rows, size_t n_rows);
    // the device copy of all instances of a DataSet, built on first use and kept with the DataSet
    static std::shared_ptr<DeviceRows> of(const DataSet &dataset);
};

class KernelMatrix {
public:
    KernelMatrix(const DataSet::node2d &instances, SvmParam param);
    // Rows `rows[0..n_rows)` of `all`, without materialising a node2d copy.
    KernelMatrix(const DataSet::node2d &all, const int *rows, size_t n_rows, SvmParam param, int repeat = 1);
    // Rows `rows[0..n_rows)` of the DataSet's device-resident instances (rows == nullptr: all of them, shared
    // in place).  The feature count is the whole DataSet's, not the subset's: extra all-zero columns add
    // exact zeros to every dot product.
    KernelMatrix(const DataSet &dataset, const int *rows, size_t n_rows, SvmParam param, int repeat = 1);

    // kernel rows of stored rows d_idx[0..m) (device, folded ids) -> element s_i*ld + j of d_out,
    // s_i = d_out_slots[i] (or i), j < n_columns(); elements are row_type() wide
    void get_rows(const int *d_idx, int m, void *d_out, int64_t ld, const int *d_out_slots = nullptr,
                  hipStream_t stream = nullptr) const;
    // the same when only the device knows how many rows there are (*d_m of at most m_max; dense layout only)
    void get_rows_counted(const int *d_idx, int m_max, const int *d_m, void *d_out, int64_t ld, const int *d_out_slots,
                          hipStream_t stream) const;
    // the m x m block K(x_idx[r], x_idx[t]) -> d_out[r*ld + t] (what the local solver reads; row_type() elements)
    void get_block(const int *d_idx, int m, void *d_out, int64_t ld, hipStream_t stream = nullptr) const;
    // kernel rows of an external batch -> element i*ld + j of d_out (row_type() elements)
    void get_rows(const DataSet::node2d &instances, void *d_out, int64_t ld) const;
    void get_rows(const std::vector<DataSet::node> *instances, size_t m, void *d_out, int64_t ld) const;   // the same for a slice

    // An external batch on the device: dense [m][lda] in the stored rows' column layout (dense stored rows only) and
    // the rows' self dot products; valid until the next call that stages a batch.  indicator_values: the stored rows
    // have indicator columns and the batch holds only zeros and ones there.
    struct StagedBatch {
        const kernel_type *a = nullptr;
        int64_t lda = 0;
        const kernel_type *sd = nullptr;
        bool indicator_values = false;
    };
    StagedBatch stage_batch(const std::vector<DataSet::node> *instances, size_t m) const;
    const DeviceRows &rows() const { return *rows_; }

    const kernel_type *diag() const { return diag_.data(); }          // device, n_instances() entries
    const kernel_type *self_dot() const { return rows_->self_dot.data(); }  // device, n_columns() entries
    size_t n_instances() const { return n_unique_ * repeat_; }        // rows of the matrix the solver sees
    size_t n_columns() const { return n_unique_; }                    // stored rows = columns of a kernel row
    int repeat() const { return repeat_; }
    int row_type() const { return param.kernel_type == SvmParam::LINEAR ? TSVM_ROW_F64 : TSVM_ROW_F32; }
    size_t row_elem_size() const { return row_type() == TSVM_ROW_F32 ? sizeof(float) : sizeof(double); }
    size_t n_features() const { return rows_->n_features; }
    size_t nnz() const { return rows_->nnz; }
    bool dense_layout() const { return rows_->dense; }
    const SvmParam &get_param() const { return param; }

    static bool choose_dense(size_t n, size_t n_features, size_t nnz);

    // Bytes the reference's SyncMem counter (syncmem.cpp:58-108) holds for its KernelMatrix of the same rows in a
    // USE_DOUBLE build: val_, col_ind_, row_ptr_, self_dot_, diag_ (kernelmatrix.cpp:211-226) and the dense and
    // sparse parts its constructor splits the columns into (CSR_DenseCSR, kernelmatrix.cpp:16-181).  This is
    // what SvmModel::get_working_set_size subtracts from the memory budget (svmmodel.cpp:437-451).  An entry
    // stored with the value 0 counts as absent in the dense layout and as a non-zero entry in the CSR layout.
    size_t reference_syncmem_bytes() const;

private:
    void finish(int repeat);

    SvmParam param;
    std::shared_ptr<DeviceRows> rows_;
    size_t n_unique_ = 0;
    int repeat_ = 1;
    tsvm::DeviceBuffer<kernel_type> diag_;
    // reusable staging for the sparse path and for external batches
    mutable tsvm::DeviceBuffer<kernel_type> stage_;
    // transposed staging of CSR working rows (get_rows / get_block), all-zero between uses; float elements when
    // the rows' values are floats
    mutable tsvm::DeviceBuffer<unsigned char> stage_w_, stage_blk_;
    mutable tsvm::DeviceBuffer<kernel_type> stage_blk_sd_;
    mutable tsvm::DeviceBuffer<kernel_type> stage_sd_;
    mutable tsvm::DeviceBuffer<kernel_type> b_val_;
    mutable tsvm::DeviceBuffer<int> b_col_;
    mutable tsvm::DeviceBuffer<int64_t> b_ptr_;
    mutable tsvm::PinnedBuffer<kernel_type> h_val_;   // host side of the batch staging
    mutable tsvm::PinnedBuffer<int> h_col_;
    mutable tsvm::PinnedBuffer<int64_t> h_ptr_;
};
