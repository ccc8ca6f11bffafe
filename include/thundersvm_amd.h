/*
 * thundersvm_amd -- C ABI of the MI355X (gfx950) back end for ThunderSVM's SMO-training and
 * kernel-evaluation path.
 *
 * Every entry point replaces one function of the reference's `svm_kernel::` namespace
 * (include/thundersvm/kernel/kernelmatrix_kernel.h:12-68, include/thundersvm/kernel/smo_kernel.h:24-45),
 * taking raw device pointers where the reference takes SyncArray<T>&.  All pointers are DEVICE
 * pointers unless a parameter is named host_*; the caller owns every buffer, the library keeps
 * none of them after the call returns.  Work is enqueued on `stream` (a hipStream_t, NULL = the
 * default stream) and is asynchronous unless stated otherwise.
 *
 * Return value: 0 on success, a positive hipError_t value for a runtime failure, a negative
 * TSVM_E* value for a rejected argument.  tsvm_last_error() describes the last failure of the
 * calling thread.  (The reference throws std::bad_alloc on out-of-memory and aborts otherwise,
 * include/thundersvm/util/common.h:33-42; the C++ wrappers above this ABI map
 * hipErrorOutOfMemory (2) to std::bad_alloc.)
 *
 * float_type and kernel_type are double (the reference built with -DUSE_DOUBLE=ON).
 */
#ifndef THUNDERSVM_AMD_H
#define THUNDERSVM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSVM_EINVAL (-1)   /* bad argument */
#define TSVM_ENOSPC (-2)   /* caller workspace too small */

/* SvmParam::KERNEL_TYPE (include/thundersvm/svmparam.h:36-38) */
enum tsvm_kernel_type { TSVM_K_LINEAR = 0, TSVM_K_POLY = 1, TSVM_K_RBF = 2, TSVM_K_SIGMOID = 3, TSVM_K_PRECOMPUTED = 4 };

/* Element type of stored kernel rows.  RBF, polynomial and sigmoid kernel values are float-rounded by
 * definition (expf / powf / tanhf in kernelmatrix_kernel.cpp:77-108, widened to kernel_type afterwards), so a
 * float row holds exactly the reference's values in half the bytes; linear kernel values are full doubles and
 * must use TSVM_ROW_F64 (the calls reject TSVM_ROW_F32 with a linear kernel).  Row strides (ld*) count elements. */
enum tsvm_row_type { TSVM_ROW_F64 = 0, TSVM_ROW_F32 = 1 };

typedef void *tsvm_stream;

const char *tsvm_last_error(void);
int tsvm_version(void);

/* ---------------------------------------------------------------------------------------------
 * KernelMatrix::get_rows / diag  (src/thundersvm/kernelmatrix.cpp:183-316)
 * ------------------------------------------------------------------------------------------- */

/* Row self dot products of a CSR matrix: self_dot[i] = sum_j val^2 in stored order
 * (KernelMatrix constructor, kernelmatrix.cpp:195-205). */
int tsvm_csr_self_dot(const double *val, const int64_t *row_ptr, int64_t n, double *self_dot, tsvm_stream stream);

/* Row self dot products of a dense row-major matrix [n][ld], over columns 0..d-1 in ascending order. */
int tsvm_dense_self_dot(const double *x, int64_t ld, int64_t n, int d, double *self_dot, tsvm_stream stream);

/* diag[i] = kappa(x_i, x_i) from the self dot products (kernelmatrix.cpp:225-247; poly_kernel /
 * sigmoid_kernel of kernelmatrix_kernel.cpp:94-108 applied to self_dot). */
int tsvm_kernel_diag(const double *self_dot, int64_t n, int kernel_type, double gamma, double coef0, int degree,
                     double *diag, tsvm_stream stream);

/* Scatter CSR rows into a zero-filled dense row-major matrix [n][ld] (column c = feature id c):
 * get_working_set_ins, kernelmatrix_kernel.cpp:9-25, applied to all rows once.  Entries with
 * col >= ld are dropped (the test-row rule of kernelmatrix.cpp:392). */
int tsvm_csr_to_dense(const double *val, const int *col, const int64_t *row_ptr, int64_t n, double *x, int64_t ld,
                      tsvm_stream stream);

/* Column statistics of the data rows (dense row-major [n][ld], columns 0..d-1; or the nnz stored entries of a CSR
 * matrix with column ids below d): counts[c] = entries of column c (dense: non-zero values; CSR: stored entries),
 * counts[d + c] = how many values of the column are neither 0 nor 1.  counts holds 2*d ints and is cleared by the call.  The per-column entry counts are what the reference's
 * KernelMatrix constructor splits the matrix by (CSR_DenseCSR, kernelmatrix.cpp:16-74). */
int tsvm_column_stats_dense(const double *x, int64_t ld, int64_t n, int d, int *counts, tsvm_stream stream);
int tsvm_column_stats_csr(const double *val, const int *col, int64_t nnz, int d, int *counts, tsvm_stream stream);

/* Dense get_rows: out[s_i*ldo + j] = kappa(a_i, x_j), i < m, j < n, where a_i is row a_idx[i] of `a`
 * (a_idx == NULL: row i) and s_i = out_slots[i] (out_slots == NULL: i) is the output row, so new kernel
 * rows can be written straight into the slots of a row cache.  x_idx != NULL restricts the columns to
 * the rows x_idx[0..n) of x (x_j = row x_idx[j]); with x_idx = a_idx = the working set this yields the
 * ws x ws block the local solver needs without touching the other n - ws rows.  Replaces get_working_set_ins + dns_csr_mul + RBF_kernel/poly_kernel/
 * sigmoid_kernel (kernelmatrix.cpp:251-312; kernelmatrix_kernel.cpp:9-25,61-108,149-160) in one
 * launch.  x is [n][ldx], a is [*][lda], both row-major fp64 with zero padding up to a multiple of
 * 8 columns (ldx % 8 == 0, lda % 8 == 0, d <= min(ldx, lda)).  The dot product is accumulated over
 * ascending column index with fused multiply-adds.  sd_x[j] / sd_a[a_idx[i]] are the self dot
 * products (used by RBF only).  out holds double or float elements as row_type says. */
int tsvm_get_rows_dense(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d, const double *sd_x, const double *a,
                        int64_t lda, const int *a_idx, int m, const double *sd_a, int kernel_type, double gamma,
                        double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                        tsvm_stream stream);

/* tsvm_get_rows_dense when the number of working rows is only known on the device: the grid is sized for m_max
 * rows, *m_dev (read by the kernel, 0 <= *m_dev <= m_max) says how many of them exist; entries of a_idx and
 * out_slots from *m_dev on are not read. */
int tsvm_get_rows_dense_counted(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d, const double *sd_x,
                                const double *a, int64_t lda, const int *a_idx, int m_max, const int *m_dev,
                                const double *sd_a, int kernel_type, double gamma, double coef0, int degree, void *out,
                                int row_type, const int *out_slots, int64_t ldo, tsvm_stream stream);

/* Indicator columns.  When the last columns of the data hold only zeros and ones (one-hot encoded categories; the
 * reference's KernelMatrix constructor moves such rarely set columns into a separate sparse part and multiplies the
 * two parts separately, kernelmatrix.cpp:58-74,318-343), the dot product over them is the number of columns both
 * rows have set.  tsvm_indicator_masks packs columns first_col .. first_col + n_cols - 1 (n_cols <= 64) of every row
 * into one 64-bit mask (bit b: column first_col + b is non-zero) and writes the largest number of set bits of a row
 * to *max_ones (device int). */
int tsvm_indicator_masks(const double *x, int64_t ld, int64_t n, int first_col, int n_cols, uint64_t *masks, int *max_ones,
                         tsvm_stream stream);

/* tsvm_get_rows_dense / tsvm_get_rows_dense_counted (m_dev != NULL) for data whose columns from d_dense on are
 * indicator columns, given as the masks of tsvm_indicator_masks (mask_x[j] for row j of x, mask_a[r] for row r of a;
 * both sides must be 0/1 there).  The matrix cores walk columns 0 .. d_dense-1 only; 1.0 is then added once per
 * indicator column set in both rows, one addition at a time, which is the serial chain of fused multiply-adds over
 * those columns bit for bit.  max_ones bounds the set bits of a row.  Results equal tsvm_get_rows_dense on all columns. */
int tsvm_get_rows_dense_indicator(const double *x, int64_t ldx, const int *x_idx, int64_t n, int d_dense, const double *sd_x,
                                  const uint64_t *mask_x, const double *a, int64_t lda, const int *a_idx, int m, const int *m_dev,
                                  const double *sd_a, const uint64_t *mask_a, int max_ones, int kernel_type, double gamma,
                                  double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                                  tsvm_stream stream);

/* Transposed dense staging of selected CSR rows: w[c*m + i] = value of feature c in row idx[i]
 * (idx == NULL: row i of the given CSR), w is [n_features][m] and is zero-filled first.
 * The sparse-path counterpart of get_working_set_ins (kernelmatrix_kernel.cpp:9-25). */
int tsvm_csr_stage_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int m,
                        int n_features, double *w, tsvm_stream stream);

/* The scatter of tsvm_csr_stage_rows without the zero fill, for a staging matrix that is kept all-zero between
 * uses: clear == 0 writes the rows' values, clear != 0 writes 0.0 to the same places (after the matrix has been
 * used).  Touches nnz entries instead of n_features x m.  w holds w_type elements (TSVM_ROW_F64 / TSVM_ROW_F32). */
int tsvm_csr_scatter_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int m,
                          int n_features, void *w, int w_type, int clear, tsvm_stream stream);

/* tsvm_get_rows_csr with the staged working rows held as w_type elements (TSVM_ROW_F64 or TSVM_ROW_F32).  Float
 * staging is exact when every value of the working rows is a float (values read from a LibSVM file or handed over
 * as float arrays are): products and sums are formed in double either way, and the kernel's time goes into
 * reading the staged rows, m elements per stored non-zero. */
int tsvm_get_rows_csr_staged(const double *val, const int *col, const int64_t *row_ptr, const int *x_idx, int64_t n,
                             const double *sd_x, const void *w, int w_type, int m, const double *sd_w, int kernel_type,
                             double gamma, double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                             tsvm_stream stream);

/* CSR get_rows: out[s_i*ldo + j] = kappa(w_i, x_j) (s_i as above) with x in CSR (n rows) and the m working rows
 * staged by tsvm_csr_stage_rows.  Accumulates over the stored order of row j's non-zeros
 * (dns_csr_mul, kernelmatrix_kernel.cpp:149-160) and applies the epilogue.  sd_w[i] are the
 * working rows' self dot products (already gathered, length m).  x_idx as in tsvm_get_rows_dense. */
int tsvm_get_rows_csr(const double *val, const int *col, const int64_t *row_ptr, const int *x_idx, int64_t n, const double *sd_x,
                      const double *w, int m, const double *sd_w, int kernel_type, double gamma, double coef0,
                      int degree, void *out, int row_type, const int *out_slots, int64_t ldo, tsvm_stream stream);

/* The CSR product on a sliced copy of the stored rows (the role of dns_csr_mul, kernelmatrix_kernel.cpp:149-160, with
 * the operands' roles exchanged: the stored rows are streamed, the working rows wait in LDS).
 * Sliced layout (sliced ELL, slices of 64 rows): entry k of row 64 s + l lies at slice_ptr[s] + 64 k + l; slice s is
 * as wide as its longest row (tsvm_csr_slice_widths gives the widths, the caller turns them into slice_ptr[s + 1] =
 * slice_ptr[s] + 64 * width[s], ceil(n / 64) + 1 entries); tsvm_csr_to_sliced fills it from the CSR arrays, padding
 * with column pad_col (= n_features) and value 0; values are stored as val_type (TSVM_ROW_F32 only when every value
 * is exactly a float).
 * tsvm_get_rows_csr_sliced: out[slot(i) * ldo + j] = kappa(row a_idx[i] of the CSR matrix (a_val, a_col, a_ptr), stored
 * row j) for i < m, j < n; sd_a is indexed by the CSR row (a_idx == NULL: rows 0 .. m-1).  Sums run over a stored row's
 * entries in stored order; entries whose feature does not occur in a block of sixteen working rows add exact zeros
 * and are skipped.  max_row_nnz: an upper bound on the entries of any working row; the working rows' block is held in
 * tsvm_get_rows_csr_sliced_lds(n_features, max_row_nnz, val_type) bytes of LDS (a table of n_features 16-bit entries
 * and a tile with a row of sixteen doubles for every feature that occurs in the block; a block with more such features
 * than the tile has rows is done in two halves): when that returns 0 the shape does not fit (eight of the longest
 * rows must) and the call is rejected (use tsvm_get_rows_csr_staged). */
int tsvm_csr_slice_widths(const int64_t *row_ptr, int64_t n, int *widths, tsvm_stream stream);
int tsvm_csr_to_sliced(const double *val, const int *col, const int64_t *row_ptr, int64_t n, const int64_t *slice_ptr, int pad_col,
                       int *ell_col, void *ell_val, int val_type, tsvm_stream stream);
size_t tsvm_get_rows_csr_sliced_lds(int n_features, int max_row_nnz, int val_type);
int tsvm_get_rows_csr_sliced(const int *ell_col, const void *ell_val, int val_type, const int64_t *slice_ptr, int64_t n,
                             const double *sd_x, const double *a_val, const int *a_col, const int64_t *a_ptr, const int *a_idx,
                             int m, const double *sd_a, int n_features, int max_row_nnz, int kernel_type, double gamma,
                             double coef0, int degree, void *out, int row_type, const int *out_slots, int64_t ldo,
                             tsvm_stream stream);

/* Device-side row subsets, so that a sub-problem (one class pair of a one-vs-one run, svc.cpp:147-150) takes its
 * rows from a data set already resident in HBM instead of a host copy:
 * dense: out row r = x row idx[r] (rows of ld doubles, ld % 4 == 0);
 * CSR: rows idx[0..m) of (val, col, row_ptr) written to (out_val, out_col) at the offsets out_ptr[0..m], which the
 * caller has computed from the row lengths. */
int tsvm_gather_rows_f64(const double *x, int64_t ld, const int *idx, int64_t m, double *out, tsvm_stream stream);
int tsvm_csr_gather_rows(const double *val, const int *col, const int64_t *row_ptr, const int *idx, int64_t m,
                         const int64_t *out_ptr, double *out_val, int *out_col, tsvm_stream stream);

/* out[t] = ids[t] % period.  The 2n-variable problem of SVR (svr.cpp:14-15) stacks the same n rows twice:
 * instance id i and i + n share one kernel row, so rows are computed, cached and stored once under the
 * folded id and are n (not 2n) columns wide. */
int tsvm_fold_ids(const int *ids, int count, int period, int *out, tsvm_stream stream);

/* out[i] = in[idx[i]] for doubles (gathers working-set self dots). */
int tsvm_gather_f64(const double *in, const int *idx, int m, double *out, tsvm_stream stream);

/* ---------------------------------------------------------------------------------------------
 * smo_kernel.cpp
 * ------------------------------------------------------------------------------------------- */

/* update_f (smo_kernel.cpp:300-319): f[j] -= sum_{t<ws, alpha_diff[t]!=0} alpha_diff[t]*K_t[j], the
 * sum taken in ascending t with fused multiply-adds.  Kernel row t starts at element
 * slots[t]*ld of k_rows (slots == NULL: slot t), so rows kept from the previous working set are
 * addressed in place instead of being copied (csmosolver.cpp:75).  Rows are n_cols wide and f has
 * n_cols*repeat entries: f[j + r*n_cols] -= (the same sum) for r < repeat, which is the reference's
 * result when its kernel matrix consists of repeat x repeat copies of one n_cols x n_cols block
 * (repeat = 2 for SVR, else 1).  ld >= n_cols rounded up to a multiple of 4 lets the kernel use
 * 16-byte loads. */
int tsvm_update_f(double *f, const double *alpha_diff, int ws_size, const void *k_rows, int row_type, const int *slots,
                  int64_t ld, int64_t n_cols, int repeat, tsvm_stream stream);

/* Bytes of device workspace tsvm_c_smo_solve / tsvm_nu_smo_solve need for a working set of ws_size. */
size_t tsvm_smo_solve_workspace(int ws_size);

/* c_smo_solve (smo_kernel.cpp:12-125).  One workgroup solves the working-set sub-problem.
 * diff[0] = initial low-up gap, diff[1] = number of inner iterations.  k_rows/slots/ld as in
 * tsvm_update_f; workspace from tsvm_smo_solve_workspace. */
int tsvm_c_smo_solve(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                     int ws_size, double Cp, double Cn, const void *k_rows, int row_type, const int *slots, int64_t ld,
                     const double *k_diag, double eps, double *diff, int max_iter, void *workspace,
                     tsvm_stream stream);

/* tsvm_c_smo_solve without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The ws x ws block goes into a static device array of 1024 x 1024 doubles (8 MiB per device, held until the
 * process ends); ws_size > 1024 is rejected with TSVM_EINVAL.  The call allocates and frees nothing.  Every call on
 * a device shares that device's array: calls that overlap on one device (different streams or threads) race, the
 * caller has to order them.  Results are those of tsvm_c_smo_solve.
 * The first call on a device looks up the array's address and the kernels' attributes (and the runtime may load the
 * library's code object then): make that call, or tsvm_c_smo_solve_static_init(), once per device outside any graph
 * capture; calls after it only launch kernels. */
int tsvm_c_smo_solve_static_init(void);
int tsvm_c_smo_solve_static(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                            int ws_size, double Cp, double Cn, const void *k_rows, int row_type, const int *slots,
                            int64_t ld, const double *k_diag, double eps, double *diff, int max_iter, tsvm_stream stream);

/* Row stride (in elements) of the ws x ws block the solver kernels read: ws rounded up to 256, 512 or 1024.
 * block_type below: element type of the block, TSVM_ROW_F64 or, when the kernel rows are float (their values are
 * floats to begin with), TSVM_ROW_F32: the same numbers in half the bytes, widened when the solver loads them. */
int tsvm_smo_solve_block_ld(int ws_size);

/* The block from stored kernel rows: kws[r*ldk + t] = element cols[t] of the row in slot slots[r] (slots == NULL:
 * slot r), r, t < ws_size, ldk = tsvm_smo_solve_block_ld(ws_size), columns t >= ws_size zero-filled; the gather that
 * replaces the strided reads k_mat_rows[row_len*i + working_set[t]] of smo_kernel.cpp:50-52,107-110. */
int tsvm_smo_gather_block(const void *k_rows, int row_type, const int *slots, int64_t ld, const int *cols, int ws_size,
                          void *kws, int block_type, tsvm_stream stream);

/* The block when slot_of_id[i] names the slot that holds instance i's row (a row cache that holds every row):
 * kws[r*ldk + t] = element ids[t] of the row in slot slot_of_id[ids[r]]; slots_out[r] receives that slot (the
 * table tsvm_update_f takes).  Nothing has to come from the host between the selection and this call. */
int tsvm_smo_gather_block_by_id(const void *k_rows, int row_type, const int *slot_of_id, int64_t ld, const int *ids,
                                int ws_size, void *kws, int block_type, int *slots_out, tsvm_stream stream);

/* Slots for the new rows of a working set, decided on the device, for a row store with a slot for every
 * instance (the reference recomputes the rows of every working set, csmosolver.cpp:65-77; rows kept here are the
 * rows get_rows would recompute).  ids_new[0..n_new) are distinct instances; those without a slot yet
 * (slot_of_id[i] < 0) take the slots state[0], state[0]+1, ... in list order.  Outputs: slot_of_id and state[0]
 * (slots in use) updated; state[1] = number of such instances, listed in miss_ids / miss_slots (the a_idx /
 * out_slots / m_dev of tsvm_get_rows_dense_counted); slots_ws[t] = slot of ids_ws[t], t < ws_size; info[0..1] =
 * state[1], state[0] (for the host: info may be pinned host memory).  Start from slot_of_id = -1, state = 0. */
int tsvm_row_slots_assign(const int *ids_new, int n_new, int *slot_of_id, int *state, int *miss_ids, int *miss_slots,
                          const int *ids_ws, int ws_size, int *slots_ws, int *info, tsvm_stream stream);

/* c_smo_solve / nu_smo_solve on a precomputed block kws[r*ldk + t] = K(x_ws[r], x_ws[t]) (ldk from
 * tsvm_smo_solve_block_ld, columns t >= ws zero or arbitrary finite values): the solver touches nothing
 * else of the kernel matrix, so it can run while the full rows are still being computed on another
 * stream.  C is passed as Cp for the nu variant (Cn unused). */
int tsvm_c_smo_solve_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                           int ws_size, double Cp, double Cn, const void *kws, int block_type, const double *k_diag, double eps,
                           double *diff, int max_iter, tsvm_stream stream);
int tsvm_nu_smo_solve_block(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                            int ws_size, double C, const void *kws, int block_type, const double *k_diag, double eps, double *diff,
                            int max_iter, tsvm_stream stream);

/* No counterpart in the reference: the two block solvers above, made to run on a chosen accelerator die (XCD, 0..7).
 * The launch has eight workgroups; under a stream whose CU mask leaves one CU per XCD one of them lands on every XCD,
 * the one on `xcd` solves, the others leave at once (whatever the placement, exactly one workgroup solves).  The local
 * solvers of up to eight class pairs can thus share one CU mask of eight CUs and still run on a CU, and behind an L2,
 * of their own.  gate: three ints of device memory, zero before the first launch, shared by the launches of one
 * stream only; epoch: 1 for the first launch on a gate, then one more per launch; gate[2] receives the XCD the
 * solver ran on. */
int tsvm_c_smo_solve_block_on_xcd(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                                  int ws_size, double Cp, double Cn, const void *kws, int block_type, const double *k_diag, double eps,
                                  double *diff, int max_iter, int *gate, int epoch, int xcd, tsvm_stream stream);
int tsvm_nu_smo_solve_block_on_xcd(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                                   int ws_size, double C, const void *kws, int block_type, const double *k_diag, double eps,
                                   double *diff, int max_iter, int *gate, int epoch, int xcd, tsvm_stream stream);

/* nu_smo_solve (smo_kernel.cpp:127-298), same conventions; diff[1] is left untouched as in the
 * reference's CPU code. */
int tsvm_nu_smo_solve(const int *y, const double *f_val, double *alpha, double *alpha_diff, const int *working_set,
                      int ws_size, double C, const void *k_rows, int row_type, const int *slots, int64_t ld,
                      const double *k_diag, double eps, double *diff, int max_iter, void *workspace,
                      tsvm_stream stream);

/* Sends ids[0 .. n_ids) (device memory, e.g. what a selection has just written) to host memory the device can write
 * (pinned and mapped: hipHostMalloc with hipHostMallocMapped, device pointer from hipHostGetDevicePointer), taken
 * modulo fold_n when fold_n > 0, and then, behind a system-wide fence, writes `word` to host_ids[word_at]
 * (word_at >= n_ids): a host thread that polls that word sees the ids once it sees the word.  It has no counterpart in
 * the reference, whose select_working_set runs on the host (csmosolver.cpp:123-165); it replaces a device-to-host copy
 * and the event behind it for callers that keep a host-side table of which kernel row lives where. */
int tsvm_report_ids(const int *ids, int n_ids, int fold_n, int *host_ids, int word_at, int word, tsvm_stream stream);

/* Bytes of device workspace tsvm_select_working_set needs for n instances. */
size_t tsvm_select_workspace(int64_t n);

/* sort_f + select_working_set fused (smo_kernel.cpp:321-332; csmosolver.cpp:123-165;
 * nusmosolver.cpp:48-118): writes into out[0..n_select) the ids the reference's alternating scan
 * over the (f, index)-sorted order would pick, skipping the ids in marked[0..n_marked).
 * nu != 0 selects the four-pointer NuSMOSolver rule.  When the candidates run out before n_select ids are found
 * (n_select larger than the number of unmarked instances) the remaining entries of out are -1: such a working set
 * must not be handed to the solver entry points, which index with every id they are given. */
int tsvm_select_working_set(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                            const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                            tsvm_stream stream);

/* The same selection for a workspace whose last use was a call of either function with the same n and nu,
 * complete on this stream or ordered before it: that call has left the workspace's counters cleared, and
 * this one skips the launch that clears them (CSMOSolver::solve, csmosolver.cpp:63-77, selects once per
 * outer iteration on the same problem).  On any other workspace content the result is undefined. */
int tsvm_select_working_set_again(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                                  const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                                  tsvm_stream stream);

/* Either selection (again == 0: any workspace content; again != 0: as tsvm_select_working_set_again) that also
 * writes the ids modulo fold_n to out_folded[0..n_select): the stored row of each selected instance when the n
 * instances are stacked copies of fold_n rows (the 2n-variable problem of SVR, svr.cpp:14-28).  Saves the separate
 * tsvm_fold_ids launch of every outer iteration. */
int tsvm_select_working_set_folded(const double *f, const int *y, const double *alpha, int64_t n, double Cp, double Cn,
                                   const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace,
                                   int again, int fold_n, int *out_folded, tsvm_stream stream);

/* tsvm_update_f followed by the selection of the next working set on the updated f, in one call: what
 * CSMOSolver::solve does at the end of one outer iteration and the start of the next (csmosolver.cpp:63-77,115-117).
 * The result is that of tsvm_update_f(f, alpha_diff, ws_size, k_rows, row_type, slots, ld, n_cols, repeat) and then
 * tsvm_select_working_set_again(f, y, alpha, n_cols * repeat, ...) (with out_folded != NULL: of
 * tsvm_select_working_set_folded with again != 0 and fold_n = n_cols).  The threads that write the new f values
 * also make the selection's first pass over the instances (keys, candidate flags, the first digit's counts), which
 * saves one pass over the instances and one launch per outer iteration.  y and alpha hold n_cols * repeat
 * entries; repeat <= 4; the workspace must be in the state tsvm_select_working_set_again asks for. */
int tsvm_update_f_select(double *f, const double *alpha_diff, int ws_size, const void *k_rows, int row_type, const int *slots,
                         int64_t ld, int64_t n_cols, int repeat, const int *y, const double *alpha, double Cp, double Cn,
                         const int *marked, int n_marked, int *out, int n_select, int nu, void *workspace, int *out_folded,
                         tsvm_stream stream);

/* ---------------------------------------------------------------------------------------------
 * predict (kernelmatrix_kernel.cpp:110-147)
 * ------------------------------------------------------------------------------------------- */

/* sum_kernel_values: dec[r*P + p] = sum_{l in SV_i} coef[(j-1)*T + l]*K[r][l]
 *                                  + sum_{l in SV_j} coef[i*T + l]*K[r][l] - rho[p]
 * for every class pair p = (i<j), P = k(k-1)/2, T = total_sv, K is [n_instances][ldk] of row_type elements. */
int tsvm_sum_kernel_values(const double *coef, int total_sv, const int *sv_start, const int *sv_count,
                           const double *rho, const void *k_mat, int row_type, int64_t ldk, double *dec_values,
                           int n_classes, int64_t n_instances, tsvm_stream stream);

/* SvmModel::predict_dec_values in one pass (src/thundersvm/model/svmmodel.cpp:74-117: KernelMatrix::get_rows of the
 * batch against the support vectors, then sum_kernel_values, kernelmatrix_kernel.cpp:110-147): the same decision
 * values, with the kernel values reduced in registers instead of being written out as a batch x support-vector
 * matrix.  Dense support vectors only.
 *
 * The caller lays the model out once: the support vectors of class s occupy the padded columns
 * [128 * T_s, 128 * T_s + n_sv[s]) where T_s = sum over earlier classes of ceil(n_sv / 128), n_pad = 128 * T_k;
 * col_map[p] = row of sv_x behind padded column p (padding: any valid row); coef_t[p * stride + c] = coefficient
 * row c (0 .. k-2, the layout of include/thundersvm/model/svmmodel.h:154-164) of that support vector, zero for
 * padding and for c >= k-1; stride = tsvm_predict_nc_stride(n_classes, d, masks given) (0: this shape is not taken,
 * use tsvm_get_rows_* and tsvm_sum_kernel_values).  chunks[2q], chunks[2q+1] = first and one-past-last 128-column
 * tile of chunk q; a chunk lies inside one class, chunks are ordered by class, class_chunk_start[s] = first chunk of
 * class s (k + 1 entries).  Each workgroup takes one chunk and 64 (d <= 128 or masks) or 128 batch rows.
 * a: the batch, dense [m][lda] in sv_x's column layout, with its rows' self dot products sd_a.  mask_sv / mask_a
 * (both or neither) and max_ones as in tsvm_get_rows_dense_indicator, d then counting the columns before the
 * indicator columns.  partial: workspace of max(n_chunks, 1) * m * (k-1) doubles.
 * dec_values[r * P + p] as tsvm_sum_kernel_values defines it; sums run over the lanes of a wavefront and over the
 * chunks in a fixed order (the reference adds the support vectors one after the other), so values agree with the
 * two-call form to rounding, not bit for bit. */
int tsvm_predict_nc_stride(int n_classes, int d, int has_masks);
int tsvm_predict_dec_values_dense(const double *sv_x, int64_t ldx, int d, const double *sd_sv, const uint64_t *mask_sv,
                                  const int *col_map, int64_t n_pad, const double *coef_t, const int *chunks,
                                  int n_chunks, const int *class_chunk_start, const double *rho, int n_classes,
                                  const double *a, int64_t lda, int64_t m, const double *sd_a, const uint64_t *mask_a,
                                  int max_ones, int kernel_type, double gamma, double coef0, int degree, double *partial,
                                  double *dec_values, tsvm_stream stream);

#ifdef __cplusplus
}
#endif
#endif
