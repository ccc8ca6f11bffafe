// The functions the reference's Python package calls (include/thundersvm_scikit.h; reference:
// src/thundersvm/thundersvm-scikit.cpp).  Marshalling only: float32 arrays in and out, the models themselves are
// the classes of models.h.  No exception leaves this file.
#include <omp.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/thundersvm_scikit.h"
#include "device.h"
#include "models.h"

namespace {

SvmModel *as_model(void *m) { return static_cast<SvmModel *>(m); }

template <typename F>
bool guarded(const char *what, F &&f) {
    try {
        std::lock_guard<std::recursive_mutex> one_at_a_time(tsvm::device_work_mutex());   // shared arena and streams
        f();
        return true;
    } catch (const std::exception &e) {
        std::fprintf(stderr, "thundersvm: %s failed: %s\n", what, e.what());
    } catch (...) {
        std::fprintf(stderr, "thundersvm: %s failed\n", what);
    }
    return false;
}

template <typename T>
void copy_out(const std::vector<T> &src, float *dst, size_t limit) {
    const size_t n = src.size() < limit ? src.size() : limit;
    for (size_t i = 0; i < n; ++i) dst[i] = (float) src[i];
}

// thundersvm-scikit.cpp:82-128 (the part both front ends share)
void train_on(DataSet &train, int svm_type, int kernel_type, int degree, float gamma, float coef0, float cost, float nu,
              float epsilon, float tol, int probability, int weight_size, const int *weight_label, const float *weight,
              int verbose, int max_iter, int n_cores, int max_mem_size, int gpu_id, int *n_features, int *n_classes,
              int *succeed, SvmModel *model) {
    succeed[0] = 1;
    tsvm::Log::enabled() = verbose != 0;
    if (n_cores > 0) omp_set_num_threads(n_cores);
    else if (n_cores != -1) std::fprintf(stderr, "thundersvm: n_jobs must be positive or -1\n");
    std::vector<int> w_label(weight_label, weight_label + (weight_size > 0 ? weight_size : 0));
    std::vector<float_type> w(weight, weight + (weight_size > 0 ? weight_size : 0));
    const bool ok = guarded("training", [&] {
        TSVM_HIP_CHECK(hipSetDevice(gpu_id));
        model->set_max_iter(max_iter);
        if (svm_type == SvmParam::NU_SVC) {   // nu must leave every class pair feasible (thundersvm-scikit.cpp:84-97)
            train.group_classes();
            for (size_t i = 0; i < train.n_classes(); ++i)
                for (size_t j = i + 1; j < train.n_classes(); ++j) {
                    const int n1 = train.count()[i], n2 = train.count()[j];
                    if (nu * (n1 + n2) / 2 > std::min(n1, n2)) {
                        std::printf("specified nu is infeasible\n");
                        succeed[0] = -1;
                    }
                }
            if (succeed[0] == -1) return;
        }
        SvmParam param;
        param.svm_type = static_cast<SvmParam::SVM_TYPE>(svm_type);
        param.kernel_type = static_cast<SvmParam::KERNEL_TYPE>(kernel_type);
        param.degree = degree;
        param.gamma = (float_type) gamma;
        param.coef0 = (float_type) coef0;
        param.C = (float_type) cost;
        param.nu = (float_type) nu;
        param.p = (float_type) epsilon;
        param.epsilon = (float_type) tol;
        param.probability = probability;
        if (max_mem_size != -1) param.max_mem_size = static_cast<size_t>(std::max(max_mem_size, 0)) << 20;
        param.nr_weight = (int) w.size();
        param.weight_label = w.empty() ? nullptr : w_label.data();
        param.weight = w.empty() ? nullptr : w.data();
        model->train(train, param);
        TSVM_LOG << "training finished";
        n_features[0] = (int) train.n_features();
        n_classes[0] = model->get_n_classes();
    });
    if (!ok) succeed[0] = -1;
}

// A failed prediction must not pass for a result: the caller's buffer is filled with NaN and the status is non-zero
// (the reference aborts the process in that case, include/thundersvm/util/common.h:38).
int predict_on(DataSet &data, SvmModel *model, float *predict_label, int verbose) {
    tsvm::Log::enabled() = verbose != 0;
    const bool ok = guarded("prediction", [&] {
        const std::vector<float_type> y = model->predict(data.instances(), -1);
        for (size_t i = 0; i < y.size(); ++i) predict_label[i] = (float) y[i];
    });
    if (!ok) std::fill(predict_label, predict_label + data.n_instances(), std::nanf(""));
    return ok ? 0 : -1;
}

void decision_on(DataSet &data, SvmModel *model, int value_size, float *dec_value) {
    const bool ok = guarded("decision values", [&] {
        model->predict(data.instances(), -1);
        copy_out(model->get_dec_value(), dec_value, (size_t) (value_size > 0 ? value_size : 0));
    });
    if (!ok) std::fill(dec_value, dec_value + (value_size > 0 ? value_size : 0), std::nanf(""));
}

}  // namespace

extern "C" {

void *model_new(int svm_type) {
    if (svm_type < SvmParam::C_SVC || svm_type > SvmParam::NU_SVR) return nullptr;
    SvmModel *m = nullptr;
    guarded("model_new", [&] { m = make_model(static_cast<SvmParam::SVM_TYPE>(svm_type)).release(); });
    return m;
}

void model_free(void *model) { delete as_model(model); }

void init_model_param(char *kernel_type, int *degree, float *gamma, float *coef0, int *probability, void *model) {
    static const char *const names[] = {"linear", "polynomial", "rbf", "sigmoid", "precomputed"};
    const SvmParam &p = as_model(model)->get_param();
    if (p.kernel_type >= 0 && p.kernel_type <= 4) std::strcpy(kernel_type, names[p.kernel_type]);
    *degree = p.degree;
    *gamma = (float) p.gamma;
    *coef0 = (float) p.coef0;
    *probability = p.probability;
}

void sparse_model_scikit(int row_size, float *val, int *row_ptr, int *col_ptr, float *label, int svm_type, int kernel_type,
                         int degree, float gamma, float coef0, float cost, float nu, float epsilon, float tol, int probability,
                         int weight_size, int *weight_label, float *weight, int verbose, int max_iter, int n_cores,
                         int max_mem_size, int gpu_id, int *n_features, int *n_classes, int *succeed, void *model) {
    DataSet train;
    if (!guarded("loading the training matrix", [&] { train.load_from_sparse(row_size, val, row_ptr, col_ptr, label); })) {
        succeed[0] = -1;
        return;
    }
    train_on(train, svm_type, kernel_type, degree, gamma, coef0, cost, nu, epsilon, tol, probability, weight_size, weight_label,
             weight, verbose, max_iter, n_cores, max_mem_size, gpu_id, n_features, n_classes, succeed, as_model(model));
}

void dense_model_scikit(int row_size, int features, float *data, float *label, int svm_type, int kernel_type, int degree,
                        float gamma, float coef0, float cost, float nu, float epsilon, float tol, int probability,
                        int weight_size, int *weight_label, float *weight, int verbose, int max_iter, int n_cores,
                        int max_mem_size, int gpu_id, int *n_features, int *n_classes, int *succeed, void *model) {
    DataSet train;
    if (!guarded("loading the training matrix", [&] { train.load_from_dense(row_size, features, data, label); })) {
        succeed[0] = -1;
        return;
    }
    train_on(train, svm_type, kernel_type, degree, gamma, coef0, cost, nu, epsilon, tol, probability, weight_size, weight_label,
             weight, verbose, max_iter, n_cores, max_mem_size, gpu_id, n_features, n_classes, succeed, as_model(model));
}

int sparse_predict(int row_size, float *val, int *row_ptr, int *col_ptr, void *model, float *predict_label, int verbose) {
    DataSet data;
    if (!guarded("loading the matrix", [&] { data.load_from_sparse(row_size, val, row_ptr, col_ptr, nullptr); })) return 0;
    return predict_on(data, as_model(model), predict_label, verbose);
}

int dense_predict(int row_size, int features, float *data_in, void *model, float *predict_label, int verbose) {
    DataSet data;
    if (!guarded("loading the matrix", [&] { data.load_from_dense(row_size, features, data_in, nullptr); })) return 0;
    return predict_on(data, as_model(model), predict_label, verbose);
}

void sparse_decision(int row_size, float *val, int *row_ptr, int *col_ptr, void *model, int value_size, float *dec_value) {
    DataSet data;
    if (!guarded("loading the matrix", [&] { data.load_from_sparse(row_size, val, row_ptr, col_ptr, nullptr); })) return;
    decision_on(data, as_model(model), value_size, dec_value);
}

void dense_decision(int row_size, int features, float *data_in, void *model, int value_size, float *dec_value) {
    DataSet data;
    if (!guarded("loading the matrix", [&] { data.load_from_dense(row_size, features, data_in, nullptr); })) return;
    decision_on(data, as_model(model), value_size, dec_value);
}

int n_sv(void *model) { return as_model(model)->total_sv(); }

void set_iter(void *model, int iter) { as_model(model)->set_max_iter(iter); }

void get_sv(int *row, int *col, float *data, int *data_size, int *sv_indices, void *model) {
    const DataSet::node2d &svs = as_model(model)->svs();
    int e = 0;
    row[0] = 0;
    for (size_t i = 0; i < svs.size(); ++i) {
        for (const DataSet::node &nd : svs[i]) {
            data[e] = (float) nd.value;
            col[e] = nd.index;
            ++e;
        }
        row[i + 1] = e;
    }
    data_size[0] = e;
    const std::vector<int> &ind = as_model(model)->get_sv_ind();
    for (size_t i = 0; i < ind.size(); ++i) sv_indices[i] = ind[i];
}

void get_support_classes(int *n_support, int n_class, void *model) {
    const std::vector<int> &c = as_model(model)->get_n_sv();
    for (int i = 0; i < n_class && i < (int) c.size(); ++i) n_support[i] = c[i];
}

void get_coef(float *dual_coef, int n_class, int n_sv_, void *model) {
    copy_out(as_model(model)->get_coef(), dual_coef, (size_t) (n_class > 1 ? n_class - 1 : 0) * (size_t) (n_sv_ > 0 ? n_sv_ : 0));
}

void get_linear_coef(float *linear_coef, int n_binary_model, int n_feature, void *model) {
    copy_out(as_model(model)->get_linear_coef(), linear_coef,
             (size_t) (n_binary_model > 0 ? n_binary_model : 0) * (size_t) (n_feature > 0 ? n_feature : 0));
}

void get_rho(float *rho_, int rho_size, void *model) {
    copy_out(as_model(model)->get_rho(), rho_, (size_t) (rho_size > 0 ? rho_size : 0));
}

void save_to_file_scikit(void *model, char *path) {
    guarded("saving the model", [&] { as_model(model)->save_to_file(path); });
}

void load_from_file_scikit(void *model, char *path) {
    guarded("loading the model", [&] { as_model(model)->load_from_file(path); });
}

char *save_to_string_scikit(void *model) {
    char *buf = nullptr;
    guarded("saving the model", [&] {
        const std::string s = as_model(model)->save_to_string();
        buf = (char *) std::malloc(s.size() + 1);
        if (buf) std::memcpy(buf, s.c_str(), s.size() + 1);
    });
    return buf;
}

void free_string(char *s) { std::free(s); }

void load_from_string_scikit(void *model, char *mstring) {
    guarded("loading the model", [&] { as_model(model)->load_from_string(mstring); });
}

void get_pro(void *model, float *prob) {
    const std::vector<float> &p = as_model(model)->get_prob_predict();
    for (size_t i = 0; i < p.size(); ++i) prob[i] = p[i];
}

void get_n_binary_models(void *model, int *n_model) { n_model[0] = as_model(model)->get_n_binary_models(); }

void get_n_classes(void *model, int *n_classes) { n_classes[0] = as_model(model)->get_n_classes(); }

void set_memory_size(void *model, int m_size) { as_model(model)->set_max_memory_size((size_t) (m_size > 0 ? m_size : 0)); }

void get_sv_max_index(void *model, int *n_feature) { n_feature[0] = as_model(model)->get_sv_max_index(); }

}  // extern "C"
