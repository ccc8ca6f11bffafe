// Model-level C ABI (include/thundersvm_amd_model.h) over the host classes.
#include <chrono>
#include "../../include/thundersvm_amd_model.h"

#include <cstring>
#include <exception>
#include <stdexcept>
#include <string>
#include <vector>
#include <new>

#include "cmdparser.h"
#include "models.h"

namespace {

thread_local std::string g_error;

struct Handle {
    std::unique_ptr<SvmModel> model;
    SolverTrace trace;
    std::vector<int64_t> sv_ptr;
};

int fail(const std::exception &e) {
    g_error = e.what();
    return dynamic_cast<const std::bad_alloc *>(&e) ? 2 : -1;
}

SvmParam to_param(const tsvm_param &p) {
    SvmParam s;
    s.svm_type = (SvmParam::SVM_TYPE) p.svm_type;
    s.kernel_type = (SvmParam::KERNEL_TYPE) p.kernel_type;
    s.degree = p.degree;
    s.gamma = p.gamma;
    s.coef0 = p.coef0;
    s.C = p.C;
    s.nu = p.nu;
    s.p = p.p;
    s.epsilon = p.epsilon;
    if (p.max_mem_size > 0) s.max_mem_size = (size_t) p.max_mem_size;
    s.nr_weight = p.nr_weight;
    s.weight_label = const_cast<int *>(p.weight_label);
    s.weight = const_cast<double *>(p.weight);
    return s;
}

}  // namespace

#define TSVM_GUARD(body)            \
    try {                           \
        std::lock_guard<std::recursive_mutex> one_at_a_time(tsvm::device_work_mutex()); \
        body;                       \
        return 0;                   \
    } catch (const std::exception &e) { \
        return fail(e);             \
    }

extern "C" {

const char *tsvm_model_last_error(void) { return g_error.c_str(); }

void *tsvm_model_new(int svm_type) {
    try {
        Handle *h = new Handle();
        h->model = make_model((SvmParam::SVM_TYPE) svm_type);
        return h;
    } catch (const std::exception &e) {
        fail(e);
        return nullptr;
    }
}

void tsvm_model_free(void *model) { delete (Handle *) model; }

static void configure(Handle *h, const tsvm_param *param, int ws_override, int keep_binary, int trace_cap, int profile) {
    tsvm::Log::enabled() = param->verbose != 0;
    h->model->set_max_iter(param->max_iter);
    h->model->ws_override = ws_override;
    h->model->keep_binary = keep_binary != 0;
    h->model->profile = profile != 0;
    h->model->cache_bytes = param->cache_bytes;
    h->model->pair_lanes = param->pair_lanes > 0 ? param->pair_lanes : 0;
    h->trace = SolverTrace();
    h->trace.cap_iters = trace_cap;
    h->model->trace_first = trace_cap > 0 ? &h->trace : nullptr;
}

int tsvm_model_train_csr(void *model, int64_t n, const int64_t *row_ptr, const int *col, const double *val,
                         const double *y, const tsvm_param *param, int ws_override, int keep_binary, int trace_cap,
                         int profile) {
    TSVM_GUARD({
        Handle *h = (Handle *) model;
        DataSet ds;
        ds.load_from_csr(n, row_ptr, col, val, y);
        configure(h, param, ws_override, keep_binary, trace_cap, profile);
        h->model->train(ds, to_param(*param));
    })
}

void *tsvm_dataset_new_csr(int64_t n, const int64_t *row_ptr, const int *col, const double *val, const double *y) {
    try {
        DataSet *ds = new DataSet();
        ds->load_from_csr(n, row_ptr, col, val, y);
        return ds;
    } catch (const std::exception &e) {
        fail(e);
        return nullptr;
    }
}

void *tsvm_dataset_load(const char *libsvm_file) {
    try {
        DataSet *ds = new DataSet();
        ds->load_from_file(libsvm_file);
        return ds;
    } catch (const std::exception &e) {
        fail(e);
        return nullptr;
    }
}

void *tsvm_dataset_load_threads(const char *libsvm_file, int n_threads) {
    try {
        DataSet *ds = new DataSet();
        ds->load_from_file(libsvm_file, n_threads);
        return ds;
    } catch (const std::exception &e) {
        fail(e);
        return nullptr;
    }
}

int64_t tsvm_dataset_info(void *dataset, int64_t *n_features, int *zero_based, int *has_labels) {
    const DataSet &ds = *(DataSet *) dataset;
    if (n_features) *n_features = (int64_t) ds.n_features();
    if (zero_based) *zero_based = ds.is_zero_based();
    if (has_labels) *has_labels = ds.y().size() == ds.n_instances();
    int64_t nnz = 0;
    for (const auto &row : ds.instances()) nnz += (int64_t) row.size();
    return nnz;
}

void tsvm_dataset_get_csr(void *dataset, int64_t *row_ptr, int *col, double *val, double *y) {
    const DataSet &ds = *(DataSet *) dataset;
    int64_t e = 0;
    for (size_t r = 0; r < ds.n_instances(); ++r) {
        if (row_ptr) row_ptr[r] = e;
        for (const auto &nd : ds.instances()[r]) {
            if (col) col[e] = nd.index;
            if (val) val[e] = nd.value;
            ++e;
        }
        if (y && r < ds.y().size()) y[r] = ds.y()[r];
    }
    if (row_ptr) row_ptr[ds.n_instances()] = e;
}

int tsvm_rule_choose_dense(int64_t n, int64_t n_features, int64_t nnz) {
    return KernelMatrix::choose_dense((size_t) n, (size_t) n_features, (size_t) nnz);
}
int tsvm_rule_indicator_run_start(const int *column_stats, int n_features) {
    return DeviceRows::indicator_run_start(column_stats, n_features);
}
int tsvm_rule_indicator_run_pays(int n_features, int first, int max_ones) {
    return DeviceRows::indicator_run_pays(n_features, first, max_ones);
}

int tsvm_dataset_to_device(void *dataset) {
    try {
        (void) DeviceRows::of(*(DataSet *) dataset);
        return 0;
    } catch (const std::exception &e) {
        return fail(e);
    }
}

void tsvm_dataset_free(void *dataset) { delete (DataSet *) dataset; }
int64_t tsvm_dataset_rows(void *dataset) { return (int64_t) ((DataSet *) dataset)->n_instances(); }

int tsvm_model_train(void *model, void *dataset, const tsvm_param *param, int ws_override, int keep_binary,
                     int trace_cap, int profile) {
    TSVM_GUARD({
        Handle *h = (Handle *) model;
        configure(h, param, ws_override, keep_binary, trace_cap, profile);
        h->model->train(*(DataSet *) dataset, to_param(*param));
    })
}

int tsvm_model_predict(void *model, void *dataset, int batch_size, double *dec_values, double *labels) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        const DataSet &ds = *(DataSet *) dataset;
        std::vector<float_type> out = m.predict(ds, batch_size);
        if (labels) memcpy(labels, out.data(), sizeof(double) * out.size());
        if (dec_values) memcpy(dec_values, m.get_dec_value().data(), sizeof(double) * m.get_dec_value().size());
    })
}

int tsvm_model_cross_validation(void *model, void *dataset, const tsvm_param *param, int n_fold, double *predictions) {
    TSVM_GUARD({
        Handle *h = (Handle *) model;
        configure(h, param, 0, 0, 0, 0);
        const DataSet &ds = *(DataSet *) dataset;
        std::vector<float_type> out = h->model->cross_validation(ds, to_param(*param), n_fold);
        memcpy(predictions, out.data(), sizeof(double) * out.size());
    })
}

int tsvm_model_train_file(void *model, const char *path, const tsvm_param *param) {
    TSVM_GUARD({
        Handle *h = (Handle *) model;
        DataSet ds;
        ds.load_from_file(path);
        configure(h, param, 0, 0, 0, 0);
        h->model->train(ds, to_param(*param));
    })
}

int tsvm_model_info(void *model, int *n_classes, int *n_binary_models, int *total_sv, int64_t *sv_nnz) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        if (n_classes) *n_classes = m.get_n_classes();
        if (n_binary_models) *n_binary_models = m.get_n_binary_models();
        if (total_sv) *total_sv = (int) m.svs().size();
        if (sv_nnz) {
            int64_t t = 0;
            for (const auto &r : m.svs()) t += (int64_t) r.size();
            *sv_nnz = t;
        }
    })
}

int tsvm_model_get(void *model, int *label, int *n_sv, double *rho, double *coef, int *sv_indices, int64_t *sv_ptr,
                   int *sv_col, double *sv_val) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        if (label && !m.get_label().empty()) memcpy(label, m.get_label().data(), sizeof(int) * m.get_label().size());
        if (n_sv) memcpy(n_sv, m.get_n_sv().data(), sizeof(int) * m.get_n_sv().size());
        if (rho) memcpy(rho, m.get_rho().data(), sizeof(double) * m.get_rho().size());
        if (coef && !m.get_coef().empty()) memcpy(coef, m.get_coef().data(), sizeof(double) * m.get_coef().size());
        if (sv_indices && !m.get_sv_ind().empty()) memcpy(sv_indices, m.get_sv_ind().data(), sizeof(int) * m.get_sv_ind().size());
        int64_t e = 0;
        if (sv_ptr) sv_ptr[0] = 0;
        for (size_t r = 0; (sv_ptr || sv_col || sv_val) && r < m.svs().size(); ++r) {
            for (const auto &nd : m.svs()[r]) {
                if (sv_col) sv_col[e] = nd.index;
                if (sv_val) sv_val[e] = nd.value;
                ++e;
            }
            if (sv_ptr) sv_ptr[r + 1] = e;
        }
    })
}

int tsvm_model_stats(void *model, int k, int64_t *n_iter, int64_t *local_iter, double *obj, double *phase_ms) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        const SolverStats &s = m.solver_stats.at(k);
        if (n_iter) *n_iter = s.n_iter;
        if (local_iter) *local_iter = s.local_iter;
        if (obj) *obj = s.obj;
        if (phase_ms) {
            phase_ms[0] = s.ms_select;
            phase_ms[1] = s.ms_get_rows;
            phase_ms[2] = s.ms_local;
            phase_ms[3] = s.ms_update_f;
            phase_ms[4] = (double) s.cache_lookups;
            phase_ms[5] = (double) s.cache_hits;
            phase_ms[6] = (double) s.cache_rows;
            phase_ms[7] = s.cache_disabled ? 1.0 : 0.0;
            phase_ms[8] = s.ms_wall;
            phase_ms[9] = s.ms_setup;
            phase_ms[10] = (double) s.ws_size;
            phase_ms[11] = (double) s.rows_computed;
            phase_ms[12] = (double) s.update_rows;
            phase_ms[13] = (double) s.solver_xcd;
            phase_ms[14] = s.ms_start;
            phase_ms[15] = s.ms_end;
        }
    })
}

int64_t tsvm_model_binary_size(void *model, int k) {
    SvmModel &m = *((Handle *) model)->model;
    return k < (int) m.binary_alpha.size() ? (int64_t) m.binary_alpha[k].size() : -1;
}

int tsvm_model_binary(void *model, int k, double *alpha_signed, double *f) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        if (alpha_signed) memcpy(alpha_signed, m.binary_alpha.at(k).data(), sizeof(double) * m.binary_alpha.at(k).size());
        if (f) memcpy(f, m.binary_f.at(k).data(), sizeof(double) * m.binary_f.at(k).size());
    })
}

int tsvm_model_trace(void *model, int *ws_size, const double **diff, const int **ws) {
    Handle *h = (Handle *) model;
    if (ws_size) *ws_size = h->trace.ws_size;
    if (diff) *diff = h->trace.diff.data();
    if (ws) *ws = h->trace.ws.data();
    return (int) (h->trace.diff.size() / 2);
}

int tsvm_model_predict_csr(void *model, int64_t nrows, const int64_t *row_ptr, const int *col, const double *val,
                           int batch_size, double *dec_values, double *labels) {
    TSVM_GUARD({
        SvmModel &m = *((Handle *) model)->model;
        DataSet ds;
        ds.load_from_csr(nrows, row_ptr, col, val, nullptr);
        std::vector<float_type> out = m.predict(ds.instances(), batch_size);
        if (labels) memcpy(labels, out.data(), sizeof(double) * (size_t) nrows);
        if (dec_values) memcpy(dec_values, m.get_dec_value().data(), sizeof(double) * m.get_dec_value().size());
    })
}

int tsvm_cmdparser_train(int argc, char **argv, tsvm_param *param, int *gamma_set, int *do_cross_validation,
                         int *nr_fold, char *input_file, char *model_file, int cap) {
    TSVM_GUARD({
        CMDParser parser;
        parser.parse_train(argc, argv, 1);
        const SvmParam &p = parser.param_cmd;
        param->svm_type = p.svm_type;
        param->kernel_type = p.kernel_type;
        param->degree = p.degree;
        param->gamma = p.gamma;
        param->coef0 = p.coef0;
        param->C = p.C;
        param->nu = p.nu;
        param->p = p.p;
        param->epsilon = p.epsilon;
        param->max_mem_size = (int64_t) p.max_mem_size;
        param->nr_weight = p.nr_weight;
        param->verbose = parser.quiet ? 0 : 1;
        if (gamma_set) *gamma_set = parser.gamma_set;
        if (do_cross_validation) *do_cross_validation = parser.do_cross_validation;
        if (nr_fold) *nr_fold = parser.nr_fold;
        if (input_file) snprintf(input_file, cap, "%s", parser.svmtrain_input_file_name.c_str());
        if (model_file) snprintf(model_file, cap, "%s", parser.model_file_name.c_str());
    })
}

int tsvm_release_device_cache(void) {
    TSVM_GUARD({ tsvm::RowArena::instance().release(); })
}

int tsvm_model_save(void *model, const char *path) {
    TSVM_GUARD({ ((Handle *) model)->model->save_to_file(path); })
}

int tsvm_model_load(void *model, const char *path) {
    TSVM_GUARD({ ((Handle *) model)->model->load_from_file(path); })
}

}  // extern "C"
