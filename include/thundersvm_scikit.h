/* The C interface the reference's Python package binds (python/thundersvm/thundersvm.py loads libthundersvm.so and
 * calls these functions through ctypes): same names, same argument lists and meanings as
 * src/thundersvm/thundersvm-scikit.cpp, exported by thundersvm_amd/libthundersvm.so.  Training and prediction run
 * on the GPU through the kernel-level ABI of thundersvm_amd.h; arrays are host memory owned by the caller.
 *
 * `model` is the opaque SvmModel* returned by model_new.  Matrices are float32: CSR as (val, row_ptr, col_ptr) with
 * zero-based column indices, dense as row-major [row_size][features].  Functions that the reference declares void
 * and that can fail here (out of memory, an unsupported option) report it through *succeed (-1) where the
 * reference has that argument, and otherwise print the reason to stderr and leave their outputs untouched. */
#ifndef THUNDERSVM_SCIKIT_H
#define THUNDERSVM_SCIKIT_H

#ifdef __cplusplus
extern "C" {
#endif

/* thundersvm-scikit.cpp:16-35.  svm_type: 0 C_SVC, 1 NU_SVC, 2 ONE_CLASS, 3 EPSILON_SVR, 4 NU_SVR; NULL for any other value. */
void *model_new(int svm_type);
void model_free(void *model);

/* thundersvm-scikit.cpp:37-39, svmmodel.cpp:463-485: parameters of a (loaded) model; kernel_type receives one of
 * "linear", "polynomial", "rbf", "sigmoid", "precomputed" (the caller provides at least 20 bytes). */
void init_model_param(char *kernel_type, int *degree, float *gamma, float *coef0, int *probability, void *model);

/* thundersvm-scikit.cpp:41-128 / 145-237: train `model` on a CSR / dense matrix.  cost = C, epsilon = the tube width p
 * of epsilon-SVR, tol = the stopping tolerance, max_mem_size in MiB (-1: default), weight_label/weight: per-class
 * factors on C, n_cores > 0 sets the OpenMP thread count of the host code, gpu_id selects the device.  Outputs:
 * n_features[0], n_classes[0], succeed[0] (1, or -1 when nu is infeasible for NU_SVC or training failed). */
void sparse_model_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *label, int svm_type, int kernel_type,
                         int degree, float gamma, float coef0, float cost, float nu, float epsilon, float tol, int probability,
                         int weight_size, int *weight_label, float *weight, int verbose, int max_iter, int n_cores,
                         int max_mem_size, int gpu_id, int *n_features, int *n_classes, int *succeed, void *model);
void dense_model_scikit(int row_size, int features, float *data, float *label, int svm_type, int kernel_type, int degree,
                        float gamma, float coef0, float cost, float nu, float epsilon, float tol, int probability,
                        int weight_size, int *weight_label, float *weight, int verbose, int max_iter, int n_cores,
                        int max_mem_size, int gpu_id, int *n_features, int *n_classes, int *succeed, void *model);

/* thundersvm-scikit.cpp:130-143 / 239-252: predicted labels (classification, one-class) or values (regression); returns 0. */
int sparse_predict(int row_size, float *val, int *row_ptr, int *col_ptr, void *model, float *predict_label, int verbose);
int dense_predict(int row_size, int features, float *data, void *model, float *predict_label, int verbose);

/* thundersvm-scikit.cpp:324-347: decision values, row_size x n_binary_models, value_size = their number. */
void sparse_decision(int row_size, float *val, int *row_ptr, int *col_ptr, void *model, int value_size, float *dec_value);
void dense_decision(int row_size, int features, float *data, void *model, int value_size, float *dec_value);

/* thundersvm-scikit.cpp:254-322: the trained model's parts.  get_sv: support vectors as CSR (row has n_sv + 1 entries,
 * col holds the one-based feature ids as stored, data_size[0] the number of stored values) and their indices in the
 * training set; get_coef: (n_class - 1) x n_sv dual coefficients; get_linear_coef: n_binary_model x n_feature weights
 * of a linear-kernel model; get_rho: rho_size values. */
int n_sv(void *model);
void set_iter(void *model, int iter);
void get_sv(int *row, int *col, float *data, int *data_size, int *sv_indices, void *model);
void get_support_classes(int *n_support, int n_class, void *model);
void get_coef(float *dual_coef, int n_class, int n_sv, void *model);
void get_linear_coef(float *linear_coef, int n_binary_model, int n_feature, void *model);
void get_rho(float *rho_, int rho_size, void *model);

/* thundersvm-scikit.cpp:349-375: LibSVM-format model text.  save_to_string_scikit returns a malloc'ed, NUL-terminated
 * copy that the caller releases with free_string. */
void save_to_file_scikit(void *model, char *path);
void load_from_file_scikit(void *model, char *path);
char *save_to_string_scikit(void *model);
void free_string(char *s);
void load_from_string_scikit(void *model, char *mstring);

/* thundersvm-scikit.cpp:377-399 */
void get_pro(void *model, float *prob);
void get_n_binary_models(void *model, int *n_model);
void get_n_classes(void *model, int *n_classes);
void set_memory_size(void *model, int m_size);
void get_sv_max_index(void *model, int *n_feature);

#ifdef __cplusplus
}
#endif
#endif
