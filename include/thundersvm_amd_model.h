/*
 * thundersvm_amd -- model-level C ABI (libthundersvm.so).
 *
 * The role the reference's extern "C" scikit layer plays for its Python binding
 * (src/thundersvm/thundersvm-scikit.cpp:15-400: model_new / *_model_scikit / get_sv / get_coef /
 * get_rho / *_decision / save / load), with float64 arrays and CSR input so that coefficients, rho
 * and decision values cross the boundary unrounded.  All pointers are HOST pointers.  A model handle
 * is an opaque SvmModel* owned by the caller (tsvm_model_new / tsvm_model_free).
 *
 * Return value: 0 on success, 2 when the device ran out of memory (the reference's std::bad_alloc),
 * -1 otherwise; tsvm_model_last_error() describes the failure.
 */
#ifndef THUNDERSVM_AMD_MODEL_H
#define THUNDERSVM_AMD_MODEL_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* SvmParam (include/thundersvm/svmparam.h:14-66) */
typedef struct tsvm_param {
    int svm_type;      /* 0 C_SVC, 1 NU_SVC, 2 ONE_CLASS, 3 EPSILON_SVR, 4 NU_SVR */
    int kernel_type;   /* 0 LINEAR, 1 POLY, 2 RBF, 3 SIGMOID, 4 PRECOMPUTED */
    int degree;
    int max_iter;      /* outer-iteration cap, -1 = none (SvmModel::set_max_iter) */
    double gamma;
    double coef0;
    double C;
    double nu;
    double p;
    double epsilon;
    int64_t max_mem_size;   /* bytes, reference default 8192 MiB */
    int nr_weight;
    int verbose;
    const int *weight_label;
    const double *weight;
    int64_t cache_bytes;    /* HBM kernel-row cache budget: -1 = nine tenths of the free device memory, 0 = off */
    int pair_lanes;         /* class pairs of a one-vs-one run in flight at a time: 0 = automatic (8 when each pair's local
                             * solver gets a compute unit of its own, else 3 pairs advanced in lockstep), 1 = one at a time */
} tsvm_param;

const char *tsvm_model_last_error(void);

void *tsvm_model_new(int svm_type);
void tsvm_model_free(void *model);

/* SvmModel::train on rows given as CSR (feature ids as in the LibSVM file, values float32-exact).
 * ws_override > 0 forces the working-set size; keep_binary keeps each binary sub-problem's alpha*y
 * and f for tsvm_model_binary; trace_cap > 0 records that many outer iterations of the first
 * sub-problem; profile != 0 times the solver phases with device events. */
int tsvm_model_train_csr(void *model, int64_t n, const int64_t *row_ptr, const int *col, const double *val,
                         const double *y, const tsvm_param *param, int ws_override, int keep_binary, int trace_cap,
                         int profile);

/* DataSet handles: rows converted once into the host layer's DataSet (DataSet::load_from_sparse's
 * role, src/thundersvm/dataset.cpp:124-148, with float64 values and the caller's feature ids), so that
 * a timed train / predict call covers what the reference's `model->train(dataset, param)` covers and
 * not the conversion.  y may be NULL for prediction-only data. */
void *tsvm_dataset_new_csr(int64_t n, const int64_t *row_ptr, const int *col, const double *val, const double *y);
void *tsvm_dataset_load(const char *libsvm_file);
/* DataSet::load_from_file (src/thundersvm/dataset.cpp:20-100) with the number of reading and parsing threads given
 * (0: what OpenMP would start, as tsvm_dataset_load and the reference do). */
void *tsvm_dataset_load_threads(const char *libsvm_file, int n_threads);
/* What a DataSet holds (for checking a loader): returns the number of stored entries; then the rows as CSR
 * (row_ptr: rows + 1 entries) with the file's feature ids, and the labels.  Any pointer may be NULL. */
int64_t tsvm_dataset_info(void *dataset, int64_t *n_features, int *zero_based, int *has_labels);
void tsvm_dataset_get_csr(void *dataset, int64_t *row_ptr, int *col, double *val, double *y);
void tsvm_dataset_free(void *dataset);
int64_t tsvm_dataset_rows(void *dataset);
/* Layout rules of the host layer, for callers that drive the kernel-level C ABI themselves and want the kernels a
 * training run would use.  choose_dense: dense row-major storage (1) or CSR (0) for n rows of n_features columns
 * with nnz stored entries (the reference decides per column, CSR_DenseCSR, src/thundersvm/kernelmatrix.cpp:16-74;
 * here one layout serves all columns).  indicator_run_start: first column of the trailing run of columns that
 * hold only zeros and ones, from the 2 * n_features counts of tsvm_column_stats_dense (n_features: none);
 * indicator_run_pays: whether get_rows leaves that run to its epilogue, given the largest number of ones a row
 * has there (tsvm_indicator_masks). */
int tsvm_rule_choose_dense(int64_t n, int64_t n_features, int64_t nnz);
int tsvm_rule_indicator_run_start(const int *column_stats, int n_features);
int tsvm_rule_indicator_run_pays(int n_features, int first, int max_ones);
/* Uploads the DataSet's rows to HBM now (dense or CSR layout, with their self dot products) instead of at the
 * first training call that uses it; the copy stays with the DataSet, and every later training call, including
 * each class pair of a one-vs-one run, takes its rows from it on the device. */
int tsvm_dataset_to_device(void *dataset);
int tsvm_model_train(void *model, void *dataset, const tsvm_param *param, int ws_override, int keep_binary,
                     int trace_cap, int profile);
int tsvm_model_predict(void *model, void *dataset, int batch_size, double *dec_values, double *labels);
/* SvmModel::cross_validation (src/thundersvm/model/svmmodel.cpp:31-71) on a freshly created model: stratified
 * n_fold folds in class order, predictions[i] = the prediction for instance i by the model trained without its
 * fold (a label for the classifiers, a value for the regressors). */
int tsvm_model_cross_validation(void *model, void *dataset, const tsvm_param *param, int n_fold, double *predictions);

/* SvmModel::train on a LibSVM text file (DataSet::load_from_file). */
int tsvm_model_train_file(void *model, const char *path, const tsvm_param *param);

int tsvm_model_info(void *model, int *n_classes, int *n_binary_models, int *total_sv, int64_t *sv_nnz);

/* get_n_sv / get_rho / get_coef / get_sv_ind / svs (svmmodel.cpp:385-411); any pointer may be NULL.
 * coef is [(n_classes-1)][total_sv] for classifiers and [total_sv] otherwise. */
int tsvm_model_get(void *model, int *label, int *n_sv, double *rho, double *coef, int *sv_indices, int64_t *sv_ptr,
                   int *sv_col, double *sv_val);

/* Solver diagnostics of binary sub-problem k: outer iterations, inner iterations, objective and
 * phase[16]: device milliseconds of select, get_rows, local solve, update_f (zeros unless profiled),
 * then kernel-row cache lookups, hits, capacity in rows, 1 if the cache was switched off, and the host
 * wall-clock milliseconds of the whole solve and of its set-up (allocations, uploads, init_f), the
 * working-set size the problem was solved with, the kernel rows computed by get_rows over the whole solve, and (when
 * profiled) the kernel rows read by update_f; then, for class pairs solved side by side, the die the pair's local solver ran
 * on (-1 otherwise), and the host clock at the start and the end of the solve (ms since the process's first solve). */
int tsvm_model_stats(void *model, int k, int64_t *n_iter, int64_t *local_iter, double *obj, double *phase_ms);

int64_t tsvm_model_binary_size(void *model, int k);
int tsvm_model_binary(void *model, int k, double *alpha_signed, double *f);

/* Recorded trajectory of the first sub-problem: returns the number of iterations recorded. */
int tsvm_model_trace(void *model, int *ws_size, const double **diff, const int **ws);

/* SvmModel::predict (svmmodel.cpp:157-171; SVC::predict svc.cpp:179-185): dec_values is
 * [nrows][n_binary_models], labels [nrows] (class label, regression value or +-1). */
int tsvm_model_predict_csr(void *model, int64_t nrows, const int64_t *row_ptr, const int *col, const double *val,
                           int batch_size, double *dec_values, double *labels);

/* CMDParser::parse_command_line for thundersvm-train (src/thundersvm/cmdparser.cpp:59-166): fills
 * *param from LibSVM-style flags; argv[0] is the program name.  in/model file names are copied into
 * the caller's buffers (each `cap` bytes).  Returns -1 with a message for an invalid command line. */
int tsvm_cmdparser_train(int argc, char **argv, tsvm_param *param, int *gamma_set, int *do_cross_validation,
                         int *nr_fold, char *input_file, char *model_file, int cap);

/* Frees the device allocation that holds kernel rows between solves (it is otherwise kept until the
 * process ends, because releasing it costs up to seconds). */
int tsvm_release_device_cache(void);

int tsvm_model_save(void *model, const char *path);
int tsvm_model_load(void *model, const char *path);

#ifdef __cplusplus
}
#endif
#endif
