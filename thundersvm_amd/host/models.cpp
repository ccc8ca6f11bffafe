#include <chrono>
#include "models.h"
#include "text_parse.h"
#include <deque>

#include <omp.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <iomanip>
#include <stdexcept>

using tsvm::abi_check;
using tsvm::DeviceBuffer;

const char *SvmParam::kernel_type_name[6] = {"linear", "polynomial", "rbf", "sigmoid", "precomputed", "NULL"};
const char *SvmParam::svm_type_name[6] = {"c_svc", "nu_svc", "one_class", "epsilon_svr", "nu_svr", "NULL"};

std::unique_ptr<SvmModel> make_model(SvmParam::SVM_TYPE type) {
    switch (type) {
        case SvmParam::C_SVC: return std::unique_ptr<SvmModel>(new SVC());
        case SvmParam::NU_SVC: return std::unique_ptr<SvmModel>(new NuSVC());
        case SvmParam::ONE_CLASS: return std::unique_ptr<SvmModel>(new OneClassSVC());
        case SvmParam::EPSILON_SVR: return std::unique_ptr<SvmModel>(new SVR());
        case SvmParam::NU_SVR: return std::unique_ptr<SvmModel>(new NuSVR());
    }
    throw std::runtime_error("unknown svm type");
}

// ------------------------------------------------------------------------------------------------
// SvmModel
// ------------------------------------------------------------------------------------------------
void SvmModel::model_setup(const DataSet &, SvmParam &p) {   // svmmodel.cpp:22-29
    n_binary_models = n_classes * (n_classes - 1) / 2;
    rho.assign(n_binary_models, 0);
    n_sv.assign(n_classes, 0);
    sv.clear();
    sv_k_mat.reset();
    predict_plan_.reset();
    sv_indices.clear();
    coef.clear();
    linear_coef.clear();
    solver_stats.clear();
    binary_alpha.clear();
    binary_f.clear();
    param = p;
    // The class weights are the caller's arrays and need not outlive this call, while the model's own copy of the
    // parameters lives as long as the model (probability_train hands it to the fold models, svc.cpp:428-462): the
    // model keeps its own copy of the two arrays and points its parameters at them.
    own_weight_label.assign(p.weight_label, p.weight_label + (p.weight_label ? p.nr_weight : 0));
    own_weight.assign(p.weight, p.weight + (p.weight ? p.nr_weight : 0));
    param.nr_weight = (int) std::min(own_weight_label.size(), own_weight.size());
    param.weight_label = param.nr_weight ? own_weight_label.data() : nullptr;
    param.weight = param.nr_weight ? own_weight.data() : nullptr;
}

static int max2power(double n) { return (int) pow(2, floor(log2f(float(n)))); }   // util/common.h:20-23

// svmmodel.cpp:437-451.  The reference subtracts the bytes its SyncMem counter holds at this point of
// train_binary (svc.cpp:147-166; svr.cpp:9-35 and the other models alike): its KernelMatrix of the problem, the
// problem's y (int), alpha and f (float_type), and `held_bytes`, what the model has kept from earlier problems
// (the alpha arrays of the class pairs already trained, svc.cpp:50-61).  The counter is restated from the
// problem's shape, not read from this build's own device allocations, so the working-set size -- and with it the
// trajectory -- is the reference's wherever its memory budget starts to bind (n + n_features above ~10^6 with the
// default 8192 MiB).  Small model members (rho, n_sv, label) are left out.
int SvmModel::get_working_set_size(const KernelMatrix &k_mat, size_t held_bytes) {
    const size_t n_instances = k_mat.n_instances(), n_features = k_mat.n_features();
    if (ws_override > 0) {
        // (a working set larger than the problem cannot be filled: the selection would hand out instance ids of -1)
        if ((size_t) ws_override > n_instances)
            throw std::invalid_argument("working-set size " + std::to_string(ws_override) + " forced on a problem of " +
                                        std::to_string(n_instances) + " instances");
        return ws_override;
    }
    const size_t used = k_mat.reference_syncmem_bytes() + n_instances * (sizeof(int) + 2 * sizeof(float_type)) + held_bytes;
    if (param.max_mem_size < used) throw std::bad_alloc();
    const size_t free_mem = param.max_mem_size - used;
    const size_t by_mem = (size_t) max2power((double) (free_mem / sizeof(kernel_type) / (n_instances + n_features)));
    const int ws = std::min(max2power((double) n_instances), (int) std::min(by_mem, (size_t) 1024));
    TSVM_LOG << "working set size = " << ws;
    return ws;
}

// sv[s] = instances[sv_indices[s]]: the model owns copies of its support vectors (svc.cpp:86-108).  With
// hundreds of thousands of support vectors the copy is tens of milliseconds of memory traffic, so it is
// spread over the host cores.
void SvmModel::copy_support_vectors(const DataSet::node2d &instances) {
    sv.resize(sv_indices.size());
#pragma omp parallel for schedule(static)
    for (size_t s = 0; s < sv_indices.size(); ++s) sv[s] = instances[sv_indices[s]];
}

void SvmModel::run_solver(CSMOSolver &solver, const KernelMatrix &k_mat, const std::vector<int> &y,
                          std::vector<float_type> &alpha, float_type &rho_out, std::vector<float_type> &f_val,
                          float_type Cp, float_type Cn, size_t held_bytes) {
    const int ws = get_working_set_size(k_mat, held_bytes);
    solver.profile = profile;
    solver.cache_bytes = cache_bytes;
    solver.trace = solver_stats.empty() ? trace_first : nullptr;
    solver.solve(k_mat, y, alpha, rho_out, f_val, param.epsilon, Cp, Cn, ws, max_iter);
    solver_stats.push_back(solver.stats);
    if (keep_binary) binary_f.push_back(f_val);
}

// Stratified folds in class order (svmmodel.cpp:31-71).
std::vector<float_type> SvmModel::cross_validation(DataSet dataset, SvmParam p, int n_fold) {
    dataset.group_classes(this->param.svm_type == SvmParam::C_SVC);
    std::vector<float_type> y_predict_all(dataset.n_instances());
    for (int k = 0; k < n_fold; ++k) {
        DataSet::node2d x_train, x_test;
        std::vector<float_type> y_train;
        std::vector<int> test_idx;
        for (size_t c = 0; c < dataset.n_classes(); ++c) {
            const int fold = dataset.count()[c] / n_fold;
            const std::vector<int> ids = dataset.original_index((int) c);
            const size_t lo = (size_t) fold * k;
            const size_t hi = (k == n_fold - 1) ? ids.size() : std::min(ids.size(), lo + fold);
            for (size_t t = 0; t < ids.size(); ++t) {
                if (t >= lo && t < hi) {
                    x_test.push_back(dataset.instances()[ids[t]]);
                    test_idx.push_back(ids[t]);
                } else {
                    x_train.push_back(dataset.instances()[ids[t]]);
                    y_train.push_back(dataset.y()[ids[t]]);
                }
            }
        }
        DataSet train_set(x_train, (int) dataset.n_features(), y_train);
        this->train(train_set, p);
        std::vector<float_type> y_predict = this->predict(x_test, 1000);
        for (size_t i = 0; i < y_predict.size(); ++i) y_predict_all[test_idx[i]] = y_predict[i];
    }
    return y_predict_all;
}

void SvmModel::compute_linear_coef_single_model(size_t n_feature, bool zero_based) {
    linear_coef.assign(zero_based ? n_feature + 1 : n_feature, 0);
    for (size_t i = 0; i < sv.size(); ++i)
        for (const auto &nd : sv[i]) linear_coef[zero_based ? nd.index : nd.index - 1] += coef[i] * nd.value;
}

// LibSVM text model (svmmodel.cpp:193-264): rho/gamma at stream default precision, coefficients with
// 16 significant digits, SV values with 8.
std::string SvmModel::save_to_string() {
    std::ostringstream s;
    s << "svm_type " << SvmParam::svm_type_name[param.svm_type] << std::endl;
    s << "kernel_type " << SvmParam::kernel_type_name[param.kernel_type] << std::endl;
    if (param.kernel_type == SvmParam::POLY) s << "degree " << param.degree << std::endl;
    if (param.kernel_type == SvmParam::POLY || param.kernel_type == SvmParam::RBF || param.kernel_type == SvmParam::SIGMOID)
        s << "gamma " << param.gamma << std::endl;
    if (param.kernel_type == SvmParam::POLY || param.kernel_type == SvmParam::SIGMOID)
        s << "coef0 " << param.coef0 << std::endl;
    s << "nr_class " << n_classes << std::endl;
    s << "total_sv " << sv.size() << std::endl;
    s << "rho ";
    for (int i = 0; i < n_binary_models; ++i) s << rho[i] << " ";
    s << std::endl;
    if (param.svm_type == SvmParam::NU_SVC || param.svm_type == SvmParam::C_SVC) {
        s << "label ";
        for (int i = 0; i < n_classes; ++i) s << label[i] << " ";
        s << std::endl << "nr_sv ";
        for (int i = 0; i < n_classes; ++i) s << n_sv[i] << " ";
        s << std::endl;
    }
    if (param.probability == 1) {
        s << "probA ";
        for (int i = 0; i < n_binary_models; ++i) s << probA[i] << " ";
        s << std::endl << "probB ";
        for (int i = 0; i < n_binary_models; ++i) s << probB[i] << " ";
        s << std::endl;
    }
    if (param.kernel_type == SvmParam::LINEAR) {
        s << "coef " << std::endl;
        for (size_t i = 0; i < linear_coef.size(); ++i) s << std::setprecision(16) << linear_coef[i] << " ";
        s << std::endl;
    }
    s << "SV " << std::endl;
    // The support-vector lines are most of a large model's text (C4: 167,298 lines, 43 MB): runs of lines are written
    // side by side into strings of their own and joined in order.  "%.16g" / "%.8g" are what the stream writes for
    // setprecision(16) / setprecision(8) (its num_put goes through the same printf conversion in the C locale).
    const int rows = (param.svm_type == SvmParam::NU_SVC || param.svm_type == SvmParam::C_SVC) ? n_classes - 1 : 1;
    const size_t n = sv.size();
    const int n_runs = (int) std::max<size_t>(1, std::min<size_t>((size_t) omp_get_max_threads() * 4, n / 256));
    std::vector<std::string> run_text(n_runs);
#pragma omp parallel for schedule(dynamic, 1)
    for (int r = 0; r < n_runs; ++r) {
        std::string &o = run_text[r];
        char buf[64];
        for (size_t i = n * r / n_runs; i < n * (r + 1) / n_runs; ++i) {
            for (int j = 0; j < rows; ++j) o.append(buf, snprintf(buf, sizeof buf, "%.16g ", (double) coef[j * n + i]));
            for (const auto &nd : sv[i]) o.append(buf, snprintf(buf, sizeof buf, "%d:%.8g ", nd.index, (double) nd.value));
            o.push_back('\n');
        }
    }
    std::string text = s.str();
    size_t total = text.size();
    for (const std::string &o : run_text) total += o.size();
    text.reserve(total);
    for (const std::string &o : run_text) text += o;
    return text;
}

void SvmModel::save_to_file(std::string path) {
    std::ofstream out(path.c_str(), std::ios_base::out | std::ios_base::trunc);
    if (!out.is_open()) throw std::runtime_error("create file " + path + " failed");
    out << save_to_string();
}

void SvmModel::load_from_file(std::string path) {
    std::ifstream in(path.c_str());
    if (!in.is_open()) throw std::runtime_error("file " + path + " not found");
    std::stringstream ss;
    ss << in.rdbuf();
    load_from_string(ss.str());
}

// svmmodel.cpp:280-383
void SvmModel::load_from_string(std::string data) {
    sv_k_mat.reset();
    predict_plan_.reset();
    std::stringstream iss(data);
    std::string key;
    while (iss >> key) {
        if (key == "svm_type") {
            std::string v;
            iss >> v;
            for (int i = 0; i < 5; ++i) if (v == SvmParam::svm_type_name[i]) param.svm_type = (SvmParam::SVM_TYPE) i;
        } else if (key == "kernel_type") {
            std::string v;
            iss >> v;
            for (int i = 0; i < 5; ++i) if (v == SvmParam::kernel_type_name[i]) param.kernel_type = (SvmParam::KERNEL_TYPE) i;
        } else if (key == "degree") {
            iss >> param.degree;
        } else if (key == "gamma") {
            iss >> param.gamma;
        } else if (key == "coef0") {
            iss >> param.coef0;
        } else if (key == "nr_class") {
            iss >> n_classes;
            n_binary_models = n_classes * (n_classes - 1) / 2;
            rho.assign(n_binary_models, 0);
            n_sv.assign(n_classes, 0);
        } else if (key == "total_sv") {
            iss >> n_total_sv;
        } else if (key == "rho") {
            for (int i = 0; i < n_binary_models; ++i) iss >> rho[i];
        } else if (key == "label") {
            label.assign(n_classes, 0);
            for (int i = 0; i < n_classes; ++i) iss >> label[i];
        } else if (key == "nr_sv") {
            for (int i = 0; i < n_classes; ++i) iss >> n_sv[i];
        } else if (key == "probA") {
            param.probability = 1;
            probA.assign(n_binary_models, 0);
            for (int i = 0; i < n_binary_models; ++i) iss >> probA[i];
        } else if (key == "probB") {
            probB.assign(n_binary_models, 0);
            for (int i = 0; i < n_binary_models; ++i) iss >> probB[i];
        } else if (key == "coef") {
            std::string line;
            std::getline(iss, line);
            std::getline(iss, line);
            std::stringstream ls(line);
            linear_coef.clear();
            float_type v;
            while (ls >> v) linear_coef.push_back(v);
        } else if (key == "SV") {
            // One line per support vector: `rows` coefficients, then index:value tokens (svmmodel.cpp:356-381).  The
            // lines are most of a large model's text: they are cut into runs of whole lines and parsed side by side,
            // each number the correctly rounded double of its text, as the stream extraction and sscanf("%lf") of the
            // reference give.  Exactly total_sv lines are read; missing ones leave empty vectors with zero coefficients.
            const bool cls = param.svm_type == SvmParam::C_SVC || param.svm_type == SvmParam::NU_SVC;
            const int rows = cls ? n_classes - 1 : 1;
            sv.assign(n_total_sv, {});
            coef.assign((size_t) rows * n_total_sv, 0);
            const char *text = data.c_str();
            const size_t size = data.size();
            size_t pos = (size_t) iss.tellg();
            const char *nl0 = pos < size ? (const char *) memchr(text + pos, '\n', size - pos) : nullptr;
            pos = nl0 ? (size_t) (nl0 - text) + 1 : size;                 // behind the rest of the "SV" line
            const int n_runs = (int) std::max<size_t>(1, std::min<size_t>((size_t) omp_get_max_threads() * 4, (size - pos) >> 16));
            std::vector<size_t> cut(n_runs + 1, size);
            cut[0] = pos;
            for (int r = 1; r < n_runs; ++r) {
                const size_t from = std::max(cut[r - 1], pos + (size - pos) / n_runs * r);
                const char *nl = from < size ? (const char *) memchr(text + from, '\n', size - from) : nullptr;
                cut[r] = nl ? (size_t) (nl - text) + 1 : size;
            }
            std::vector<size_t> first_line(n_runs + 1, 0);                // lines (newlines) before each run
#pragma omp parallel for schedule(static, 1)
            for (int r = 0; r < n_runs; ++r) {
                size_t c = 0;
                for (const char *q = text + cut[r], *e = text + cut[r + 1]; q < e; ++c) {
                    const char *nl = (const char *) memchr(q, '\n', e - q);
                    if (!nl) break;
                    q = nl + 1;
                }
                first_line[r + 1] = c;
            }
            for (int r = 0; r < n_runs; ++r) first_line[r + 1] += first_line[r];
            std::vector<int> run_max(n_runs, 0);
            std::vector<char> run_bad(n_runs, 0);
#pragma omp parallel for schedule(dynamic, 1)
            for (int r = 0; r < n_runs; ++r) {
                const char *q = text + cut[r], *e = text + cut[r + 1];
                std::vector<DataSet::node> row;
                for (size_t i = first_line[r]; q < e && i < (size_t) n_total_sv; ++i) {
                    const char *eol = (const char *) memchr(q, '\n', e - q);
                    if (!eol) eol = e;
                    const char *t;
                    for (int j = 0; j < rows; ++j) {
                        while (q < eol && tsvm::is_blank(*q)) ++q;
                        if (q >= eol) break;                              // a short line: the other coefficients stay 0
                        coef[(size_t) j * n_total_sv + i] = tsvm::parse_double(q, eol, &t);
                        if (t == q) { run_bad[r] = 1; break; }
                        q = t;
                    }
                    row.clear();
                    while (!run_bad[r]) {
                        while (q < eol && tsvm::is_blank(*q)) ++q;
                        if (q >= eol) break;
                        char *after;
                        const long idx = strtol(q, &after, 10);
                        if (after == q || after >= eol || *after != ':') { run_bad[r] = 1; break; }
                        q = after + 1;
                        if (q >= eol || tsvm::is_blank(*q)) { run_bad[r] = 1; break; }   // "index:" without a value
                        const double v = tsvm::parse_double(q, eol, &t);
                        if (t == q) { run_bad[r] = 1; break; }
                        q = t;
                        row.emplace_back((int) idx, v);
                        run_max[r] = std::max(run_max[r], (int) idx);
                    }
                    if (run_bad[r]) break;
                    sv[i].assign(row.begin(), row.end());
                    q = eol + 1;
                }
            }
            for (int r = 0; r < n_runs; ++r) {
                if (run_bad[r]) throw std::runtime_error("error when loading model file");
                sv_max_index = std::max(sv_max_index, run_max[r]);
            }
            break;                                                        // nothing follows the support vectors
        }
    }
    if (param.svm_type != SvmParam::C_SVC && param.svm_type != SvmParam::NU_SVC) {
        n_sv.assign(2, 0);
        n_sv[0] = n_total_sv;
    }
}

// ------------------------------------------------------------------------------------------------
// SVC (svc.cpp)
// ------------------------------------------------------------------------------------------------
void SVC::model_setup(const DataSet &dataset, SvmParam &p) {   // svc.cpp:16-39
    n_classes = (int) dataset.n_classes();
    label = dataset.label();
    SvmModel::model_setup(dataset, p);
    param.svm_type = SvmParam::C_SVC;
    c_weight.assign(n_classes, 1);
    for (int w = 0; w < p.nr_weight; ++w) {
        bool found = false;
        for (int c = 0; c < n_classes && !found; ++c)
            if (p.weight_label[w] == label[c]) { c_weight[c] *= p.weight[w]; found = true; }
        if (!found) TSVM_LOG << "weighted label " << p.weight_label[w] << " not found";
    }
}

void SVC::train(const DataSet &dataset, SvmParam p) {   // svc.cpp:41-145
    // the reference groups a copy of the data set (svc.cpp:42-43); grouping only reads y, so the copy
    // here shares nothing but the labels and the instances are referenced in place
    DataSet grouped = dataset.grouped_view();
    model_setup(grouped, p);
    const int n = (int) grouped.n_instances();
    std::vector<std::vector<float_type>> alpha(n_binary_models);
    std::vector<char> is_sv(n, 0);
    int k = 0;
    // pairs in flight: up to eight when every pair's solver gets a CU of its own and the pairs advance independently
    // (train_pairs_in_lockstep), three when the pairs alternate between a solver phase and a chip-wide phase
    const int lanes = std::min(pair_lanes > 0 ? pair_lanes : SolveTask::cu_split_available() ? 8 : 3, n_binary_models);
    if (lanes > 1 && !profile && !trace_first) {
        train_pairs_in_lockstep(grouped, lanes, alpha);
    } else {
        size_t held = 0;   // alpha arrays of the pairs already trained (svc.cpp:50-61 keeps them to the end)
        for (int i = 0; i < n_classes; ++i)
            for (int j = i + 1; j < n_classes; ++j, ++k) {
                BinaryProblem p;
                p.k = k;
                setup_binary(grouped, i, j, p);
                run_solver(*p.solver, *p.k_mat, p.y, p.alpha, rho[k], p.f_val, p.Cp, p.Cn, held);
                held += p.y.size() * sizeof(float_type);
                finish_binary(p, alpha[k]);
            }
    }
    // (the pairs' parts of what follows are independent of one another: one host thread per pair)
    std::vector<std::pair<int, int>> pair_of;
    for (int i = 0; i < n_classes; ++i)
        for (int j = i + 1; j < n_classes; ++j) pair_of.push_back({i, j});
#pragma omp parallel for schedule(dynamic, 1)
    for (int kk = 0; kk < n_binary_models; ++kk) {
        const std::vector<int> ids = grouped.original_index(pair_of[kk].first, pair_of[kk].second);
        for (size_t l = 0; l < ids.size(); ++l)
            if (alpha[kk][l] != 0) __atomic_store_n(&is_sv[ids[l]], (char) 1, __ATOMIC_RELAXED);   // several pairs may mark one instance
    }
    if (keep_binary)
        for (int kk = 0; kk < n_binary_models; ++kk) binary_alpha.push_back(alpha[kk]);
    // support vectors class by class, in grouped order
    for (int c = 0; c < n_classes; ++c)
        for (int id : grouped.original_index(c))
            if (is_sv[id]) {
                n_sv[c]++;
                sv_indices.push_back(id);
            }
    copy_support_vectors(grouped.instances());
    n_total_sv = (int) sv.size();
    TSVM_LOG << "#total unique sv = " << n_total_sv;
    // LibSVM coefficient layout: pair (i<j) stores class i's SVs in row j-1 and class j's SVs in row i
    coef.assign((size_t) (n_classes - 1) * n_total_sv, 0);
    std::vector<int> sv_start(n_classes, 0);
    for (int c = 1; c < n_classes; ++c) sv_start[c] = sv_start[c - 1] + n_sv[c - 1];
#pragma omp parallel for schedule(dynamic, 1)
    for (int kk = 0; kk < n_binary_models; ++kk) {   // (every pair writes two segments of coef that no other pair writes)
        const int i = pair_of[kk].first, j = pair_of[kk].second;
        const std::vector<int> ids = grouped.original_index(i, j);
        const int ci = grouped.count()[i];
        int at = sv_start[i];
        for (int l = 0; l < ci; ++l)
            if (is_sv[ids[l]]) coef[(size_t) (j - 1) * n_total_sv + at++] = alpha[kk][l];
        at = sv_start[j];
        for (size_t l = ci; l < ids.size(); ++l)
            if (is_sv[ids[l]]) coef[(size_t) i * n_total_sv + at++] = alpha[kk][l];
    }
    if (param.kernel_type == SvmParam::LINEAR) {   // explicit w per pair (svc.cpp:111-135)
        const size_t nf = grouped.n_features();
        linear_coef.assign((size_t) n_binary_models * (grouped.is_zero_based() ? nf + 1 : nf), 0);
        k = 0;
        for (int i = 0; i < n_classes; ++i)
            for (int j = i + 1; j < n_classes; ++j, ++k) {
                const std::vector<int> ids = grouped.original_index(i, j);
                for (size_t l = 0; l < ids.size(); ++l) {
                    if (alpha[k][l] == 0) continue;
                    for (const auto &nd : grouped.instances()[ids[l]])
                        linear_coef[k * nf + (grouped.is_zero_based() ? nd.index : nd.index - 1)] += alpha[k][l] * nd.value;
                }
            }
    }
    if (param.probability == 1) {   // svc.cpp:137-143
        TSVM_LOG << "performing probability train";
        probA.assign(n_binary_models, 0);
        probB.assign(n_binary_models, 0);
        probability_train(grouped);
    }
}

void SVC::setup_binary(const DataSet &dataset, int i, int j, BinaryProblem &p) {   // svc.cpp:147-170
    const std::vector<int> ids = dataset.original_index(i, j);
    const int ci = dataset.count()[i], n = (int) ids.size();
    p.i = i;
    p.j = j;
    p.y.resize(n);
    p.f_val.resize(n);
    p.alpha.assign(n, 0);
    for (int l = 0; l < n; ++l) {
        p.y[l] = l < ci ? +1 : -1;
        p.f_val[l] = l < ci ? -1 : +1;
    }
    p.k_mat.reset(new KernelMatrix(dataset, ids.data(), ids.size(), param));
    p.solver.reset(new CSMOSolver());
    p.Cp = param.C * c_weight[i];
    p.Cn = param.C * c_weight[j];
}

void SVC::finish_binary(BinaryProblem &p, std::vector<float_type> &alpha_out) {   // svc.cpp:171-177
    int count = 0;
    for (size_t l = 0; l < p.alpha.size(); ++l) {
        p.alpha[l] *= p.y[l];
        if (p.alpha[l] != 0) count++;
    }
    TSVM_LOG << "rho = " << rho[p.k] << ", #sv = " << count;
    alpha_out = std::move(p.alpha);
}

// The class pairs are independent problems.  Up to `lanes` of them are in flight, each a SolveTask with its own
// slice of the kernel-row arena; a pair that finishes hands its lane to another pair, and the result of a pair
// depends neither on what runs beside it nor on when it runs.  When every lane's local solver has a compute unit
// of its own, the lanes advance independently.  Otherwise the pairs advance one outer iteration at a time in
// three phases separated by events: (1) selection, kernel rows and the solver's block of every pair, (2) the
// local solvers of all pairs, single workgroups that run side by side on different CUs, (3) update_f of every
// pair, so that no chip-wide kernel shares CUs with a local solver (next to one, each solver iteration takes
// two to three times longer).
//
// Which pair runs when, and on how much of the arena.  The pairs are taken largest first, so that the run does not end
// on one long pair with the other lanes idle.  What a pair gains from the arena depends on its size: a "small" pair,
// one whose whole kernel matrix fits an equal share of the budget, needs exactly that much and then computes every row
// once; a large pair hits in proportion to the slots it gets.  One lane therefore gets a slice that holds the
// largest small pair and works through the small pairs; the other lanes share the rest of the budget and take the
// large pairs, then whatever small pairs are left.  (Measured on seven classes of 2,400 to 246,000 instances with
// eight lanes: 1.87 s; with equal slices in the reference's order 1.93 s; with three large lanes and five small
// ones 2.35 s: the large pairs are what the time goes into, and they advance at a rate that hardly depends on
// how many of them share the chip, so long as there are at least five.)
void SVC::train_pairs_in_lockstep(const DataSet &grouped, int lanes, std::vector<std::vector<float_type>> &alpha) {
    struct PairId { int i, j; };
    std::vector<PairId> pairs;
    for (int i = 0; i < n_classes; ++i)
        for (int j = i + 1; j < n_classes; ++j) pairs.push_back({i, j});
    const size_t esz = param.kernel_type == SvmParam::LINEAR ? sizeof(double) : sizeof(float);
    tsvm::RowArena &arena = tsvm::RowArena::instance();
    const size_t budget = cache_bytes > 0 ? (size_t) cache_bytes : cache_bytes < 0 ? arena.auto_budget() : 0;
    // per pair: bytes of its working-set rows (the least a slice must hold) and of its whole kernel matrix
    std::vector<size_t> ws_bytes(pairs.size()), full_bytes(pairs.size());
    std::vector<int> by_size(pairs.size());
    for (size_t k = 0; k < pairs.size(); ++k) {
        const size_t cols = (size_t) grouped.count()[pairs[k].i] + grouped.count()[pairs[k].j];
        const size_t ld = (cols + 7) / 8 * 8;
        ws_bytes[k] = (size_t) 1024 * ld * esz;
        full_bytes[k] = std::max(cols * ld * esz, ws_bytes[k]);
        by_size[k] = (int) k;
    }
    std::stable_sort(by_size.begin(), by_size.end(), [&](int a, int b) { return full_bytes[a] > full_bytes[b]; });
    const bool two_kinds = SolveTask::cu_split_available();   // (the lockstep schedule keeps equal lanes and the reference's order)
    std::deque<int> large_q, small_q;
    size_t need_min = 0, small_slice = 0;
    for (int k : by_size) {
        need_min = std::max(need_min, ws_bytes[k]);
        if (two_kinds && full_bytes[k] <= budget / lanes) {
            small_q.push_back(k);
            small_slice = std::max(small_slice, full_bytes[k]);
        } else {
            large_q.push_back(k);
        }
    }
    int n_large_lanes, n_small_lanes;
    if (!two_kinds) {
        large_q.assign(by_size.size(), 0);
        for (size_t k = 0; k < pairs.size(); ++k) large_q[k] = (int) k;
        n_large_lanes = lanes;
        n_small_lanes = 0;
    } else if (small_q.empty()) {
        n_large_lanes = std::min<int>((int) large_q.size(), std::min(lanes, 4));
        n_small_lanes = 0;
    } else if (large_q.empty()) {
        n_large_lanes = 0;
        n_small_lanes = std::min<int>((int) small_q.size(), lanes);
    } else {
        n_large_lanes = std::min<int>((int) large_q.size(), std::max(1, lanes - 1));
        n_small_lanes = std::min<int>((int) small_q.size(), lanes - n_large_lanes);
    }
    lanes = n_large_lanes + n_small_lanes;
    small_slice = (small_slice + 255) / 256 * 256;
    size_t large_slice = 0;
    if (n_large_lanes > 0) {
        const size_t left = budget > small_slice * n_small_lanes ? budget - small_slice * n_small_lanes : 0;
        large_slice = std::max(left / n_large_lanes / 256 * 256, (need_min + 255) / 256 * 256);   // never above the budget: the arena would be re-allocated
    }
    // lanes 0 .. n_large_lanes-1 are the large ones
    std::vector<size_t> slice_at(lanes + 1, 0);
    for (int l = 0; l < lanes; ++l) slice_at[l + 1] = slice_at[l] + (l < n_large_lanes ? large_slice : small_slice);
    char *const pool = (char *) arena.acquire(slice_at[lanes], cache_bytes < 0);

    // what the reference still holds of the pairs trained before pair k when it sizes pair k's working set: their
    // alpha arrays (svc.cpp:50-61), whatever runs beside pair k here
    std::vector<size_t> alpha_bytes_before(pairs.size() + 1, 0);
    for (size_t k = 0; k < pairs.size(); ++k)
        alpha_bytes_before[k + 1] = alpha_bytes_before[k] +
                                    ((size_t) grouped.count()[pairs[k].i] + grouped.count()[pairs[k].j]) * sizeof(float_type);
    solver_stats.assign(pairs.size(), SolverStats());
    if (keep_binary) binary_f.assign(pairs.size(), std::vector<float_type>());
    std::vector<std::unique_ptr<BinaryProblem>> active;
    std::vector<int> free_lanes;
    for (int l = 0; l < lanes; ++l) free_lanes.push_back(l);
    // the pair a free lane should run next (-1: none)
    auto next_for = [&](int lane) {
        std::deque<int> &mine = lane < n_large_lanes ? large_q : small_q;
        std::deque<int> &q = !mine.empty() ? mine : lane < n_large_lanes ? small_q : mine;
        if (q.empty()) return -1;
        const int k = q.front();
        q.pop_front();
        return k;
    };
    auto start_on = [&](int lane, int k) {
        std::unique_ptr<BinaryProblem> p(new BinaryProblem());
        p->k = k;
        setup_binary(grouped, pairs[k].i, pairs[k].j, *p);
        p->lane = lane;
        const int ws = get_working_set_size(*p->k_mat, alpha_bytes_before[p->k]);
        p->solver->cache_bytes = cache_bytes;
        p->task.reset(new SolveTask(*p->solver, *p->k_mat, p->y, p->alpha, rho[p->k], p->f_val, param.epsilon, p->Cp, p->Cn, ws,
                                    max_iter, pool + slice_at[lane], slice_at[lane + 1] - slice_at[lane], lane, lanes));
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&p->rows_done, hipEventDisableTiming));
        TSVM_HIP_CHECK(hipEventCreateWithFlags(&p->solved, hipEventDisableTiming));
        active.push_back(std::move(p));
    };
    // gives every free lane that can still get a pair one; returns how many were started
    auto start_more = [&]() {
        int n_started = 0;
        for (size_t f = 0; f < free_lanes.size();) {
            const int k = next_for(free_lanes[f]);
            if (k < 0) { ++f; continue; }
            const int lane = free_lanes[f];
            free_lanes.erase(free_lanes.begin() + f);
            start_on(lane, k);
            ++n_started;
        }
        return n_started;
    };
    auto retire = [&](size_t a) {
        BinaryProblem &p = *active[a];
        solver_stats[p.k] = p.task->stats();
        if (keep_binary) binary_f[p.k] = p.f_val;
        p.task.reset();   // synchronises and releases the pair's stream before its lane is reused
        (void) hipEventDestroy(p.rows_done);
        (void) hipEventDestroy(p.solved);
        finish_binary(p, alpha[p.k]);
        free_lanes.push_back(p.lane);
        active.erase(active.begin() + a);
    };
    start_more();
    if (!active.empty() && active.front()->task->split_streams()) {
        // Every pair's solver has CUs of its own, so the pairs need no common phases: each lane runs at its own
        // pace.  The host looks at the lanes in turn and serves whichever has something to do: a lane whose
        // iteration has reported gets its next selection, block and solver enqueued; a lane whose new ids have
        // arrived (host-side row cache) gets its rows and update_f.  A small pair next to a large one thus makes
        // several iterations in the time the large one makes one.
        auto begin_iteration = [](BinaryProblem &p) {
            p.task->enqueue_select();
            p.task->enqueue_block();
            p.task->enqueue_solver();
            p.rows_pending = true;
        };
        for (auto &p : active) begin_iteration(*p);
        while (!active.empty()) {
            bool served = false;
            for (size_t a = 0; a < active.size();) {
                BinaryProblem &p = *active[a];
                if (p.rows_pending) {
                    if (p.task->rows_ready()) {
                        p.task->enqueue_rows();
                        p.task->enqueue_update();
                        p.rows_pending = false;
                        served = true;
                    }
                    ++a;
                } else if (p.task->iteration_done()) {
                    served = true;
                    if (p.task->finish_iteration()) {
                        retire(a);
                        const size_t before = active.size();
                        start_more();
                        for (size_t b = before; b < active.size(); ++b) begin_iteration(*active[b]);
                    } else {
                        begin_iteration(p);
                        ++a;
                    }
                } else {
                    ++a;
                }
            }
            if (!served) __builtin_ia32_pause();
        }
        return;
    }
    while (!active.empty()) {
        for (auto &p : active) p->task->enqueue_select();
        {
        for (auto &p : active) {
            p->task->enqueue_rows();
            p->task->enqueue_block();
            TSVM_HIP_CHECK(hipEventRecord(p->rows_done, p->task->stream()));
        }
        for (auto &p : active) {
            for (auto &o : active)
                if (o.get() != p.get()) TSVM_HIP_CHECK(hipStreamWaitEvent(p->task->stream(), o->rows_done, 0));
            p->task->enqueue_solver();
            TSVM_HIP_CHECK(hipEventRecord(p->solved, p->task->stream()));
        }
        for (auto &p : active) {
            for (auto &o : active)
                if (o.get() != p.get()) TSVM_HIP_CHECK(hipStreamWaitEvent(p->task->stream(), o->solved, 0));
            p->task->enqueue_update();
        }
        }
        for (size_t a = 0; a < active.size();) {
            if (!active[a]->task->finish_iteration()) { ++a; continue; }
            retire(a);
        }
        start_more();
    }
}

std::vector<float_type> SVC::finish_predict(int n_instances) {   // svc.cpp:179-185
    return predict_label(dec_values, n_instances);
}

// ------------------------------------------------------------------------------------------------
// Probability estimates (svc.cpp:197-491): Platt scaling of every pair's decision values, fitted on
// decision values from a 5-fold cross-validation, and pairwise coupling of the pair probabilities
// (Lin, Lin, Weng, "A note on Platt's probabilistic outputs for support vector machines", 2007; Wu, Lin,
// Weng, "Probability estimates for multi-class classification by pairwise coupling", 2004).
// ------------------------------------------------------------------------------------------------
namespace {

// P(y = +1 | dec) = 1 / (1 + exp(A*dec + B)), in the form that avoids cancellation (svc.cpp:197-204)
float_type sigmoid_predict(float_type dec, float_type A, float_type B) {
    const double v = dec * A + B;
    return v >= 0 ? exp(-v) / (1.0 + exp(-v)) : 1.0 / (1 + exp(v));
}

// negative log likelihood of the targets t under the sigmoid with parameters (A, B)
double sigmoid_objective(const std::vector<float_type> &dec, const std::vector<double> &t, double A, double B) {
    double f = 0.0;
    for (size_t i = 0; i < dec.size(); ++i) {
        const double v = dec[i] * A + B;
        f += v >= 0 ? t[i] * v + log(1 + exp(-v)) : (t[i] - 1) * v + log(1 + exp(v));
    }
    return f;
}

// Newton's method with backtracking on (A, B) (svc.cpp:318-430)
void sigmoid_train(const std::vector<float_type> &dec, const std::vector<int> &labels, float_type &A, float_type &B) {
    const size_t l = dec.size();
    double prior1 = 0, prior0 = 0;
    for (size_t i = 0; i < l; ++i) (labels[i] > 0 ? prior1 : prior0) += 1;
    const int max_iter = 100;
    const double min_step = 1e-10, sigma = 1e-12, eps = 1e-5;
    const double hi_target = (prior1 + 1.0) / (prior1 + 2.0), lo_target = 1 / (prior0 + 2.0);
    std::vector<double> t(l);
    for (size_t i = 0; i < l; ++i) t[i] = labels[i] > 0 ? hi_target : lo_target;
    A = 0.0;
    B = log((prior0 + 1.0) / (prior1 + 1.0));
    double fval = sigmoid_objective(dec, t, A, B);
    int iter = 0;
    for (; iter < max_iter; ++iter) {
        double h11 = sigma, h22 = sigma, h21 = 0.0, g1 = 0.0, g2 = 0.0;   // H + sigma*I keeps the Hessian positive definite
        for (size_t i = 0; i < l; ++i) {
            const double v = dec[i] * A + B;
            double pp, qq;
            if (v >= 0) { pp = exp(-v) / (1.0 + exp(-v)); qq = 1.0 / (1.0 + exp(-v)); }
            else { pp = 1.0 / (1.0 + exp(v)); qq = exp(v) / (1.0 + exp(v)); }
            const double d2 = pp * qq, d1 = t[i] - pp;
            h11 += dec[i] * dec[i] * d2;
            h22 += d2;
            h21 += dec[i] * d2;
            g1 += dec[i] * d1;
            g2 += d1;
        }
        if (fabs(g1) < eps && fabs(g2) < eps) break;
        const double det = h11 * h22 - h21 * h21;
        const double dA = -(h22 * g1 - h21 * g2) / det, dB = -(-h21 * g1 + h11 * g2) / det;
        const double gd = g1 * dA + g2 * dB;
        double step = 1;
        while (step >= min_step) {
            const double newA = A + step * dA, newB = B + step * dB;
            const double newf = sigmoid_objective(dec, t, newA, newB);
            if (newf < fval + 0.0001 * step * gd) {   // sufficient decrease
                A = newA;
                B = newB;
                fval = newf;
                break;
            }
            step = step / 2.0;
        }
        if (step < min_step) {
            printf("Line search fails in two-class probability estimates\n");
            break;
        }
    }
    if (iter >= max_iter) printf("Reaching maximal iterations in two-class probability estimates\n");
}

}  // namespace

// Class probabilities p from the pairwise r[i][j] = P(class i | class i or j): the fixed-point iteration for
// min sum_{i<j} (r[j][i]*p[i] - r[i][j]*p[j])^2 subject to sum p = 1 (svc.cpp:206-263).
void SVC::multiclass_probability(const std::vector<std::vector<float_type>> &r, std::vector<float_type> &p) const {
    const int k = n_classes;
    const int max_it = std::max(100, k);
    std::vector<std::vector<double>> Q(k, std::vector<double>(k, 0.0));
    std::vector<double> Qp(k);
    const double eps = 0.005 / k;
    for (int t = 0; t < k; ++t) {
        p[t] = 1.0 / k;
        Q[t][t] = 0;
        for (int j = 0; j < t; ++j) {
            Q[t][t] += r[j][t] * r[j][t];
            Q[t][j] = Q[j][t];
        }
        for (int j = t + 1; j < k; ++j) {
            Q[t][t] += r[j][t] * r[j][t];
            Q[t][j] = -r[j][t] * r[t][j];
        }
    }
    int iter = 0;
    for (; iter < max_it; ++iter) {
        double pQp = 0;   // recomputed every sweep for accuracy
        for (int t = 0; t < k; ++t) {
            Qp[t] = 0;
            for (int j = 0; j < k; ++j) Qp[t] += Q[t][j] * p[j];
            pQp += p[t] * Qp[t];
        }
        double max_error = 0;
        for (int t = 0; t < k; ++t) max_error = std::max(max_error, fabs(Qp[t] - pQp));
        if (max_error < eps) break;
        for (int t = 0; t < k; ++t) {
            const double diff = (-Qp[t] + pQp) / Q[t][t];
            p[t] += diff;
            pQp = (pQp + diff * (diff * Q[t][t] + 2 * Qp[t])) / (1 + diff) / (1 + diff);
            for (int j = 0; j < k; ++j) {
                Qp[j] = (Qp[j] + diff * Q[t][j]) / (1 + diff);
                p[j] /= (1 + diff);
            }
        }
    }
    if (iter >= max_it) printf("Exceeds max_iter in multiclass_prob\n");
}

// probA / probB of every class pair from out-of-fold decision values.  Five folds cut class by class from the
// grouped order (the last fold takes the remainder); every fold trains a plain C-SVC model with the same
// parameters, as the reference does also when the model being trained is a NuSVC.
void SVC::probability_train(const DataSet &grouped) {
    SvmParam param_no_prob = param;
    param_no_prob.probability = 0;
    const int n_fold = 5;
    std::vector<float_type> dec_all(grouped.n_instances() * (size_t) n_binary_models);
    for (int fold = 0; fold < n_fold; ++fold) {
        DataSet::node2d x_train, x_test;
        std::vector<float_type> y_train;
        std::vector<int> test_idx;
        for (size_t c = 0; c < grouped.n_classes(); ++c) {
            const std::vector<int> ids = grouped.original_index((int) c);
            const size_t per_fold = ids.size() / n_fold;
            const size_t begin = per_fold * fold;
            const size_t end = fold == n_fold - 1 ? ids.size() : std::min(ids.size(), begin + per_fold);
            for (size_t l = 0; l < ids.size(); ++l) {
                if (l >= begin && l < end) {
                    x_test.push_back(grouped.instances()[ids[l]]);
                    test_idx.push_back(ids[l]);
                } else {
                    x_train.push_back(grouped.instances()[ids[l]]);
                    y_train.push_back(grouped.y()[ids[l]]);
                }
            }
        }
        SVC fold_model;
        fold_model.set_max_iter(max_iter);
        fold_model.cache_bytes = cache_bytes;
        fold_model.pair_lanes = pair_lanes;
        fold_model.train(DataSet(x_train, (int) grouped.n_features(), y_train), param_no_prob);
        std::vector<float_type> dec;
        fold_model.predict_dec_values(x_test, dec, 1000);
        for (size_t t = 0; t < x_test.size(); ++t)
            std::copy(dec.begin() + t * n_binary_models, dec.begin() + (t + 1) * n_binary_models,
                      dec_all.begin() + (size_t) test_idx[t] * n_binary_models);
    }
    int k = 0;
    for (int i = 0; i < n_classes; ++i)
        for (int j = i + 1; j < n_classes; ++j, ++k) {
            std::vector<int> y;
            std::vector<float_type> dec_pair;
            for (int side = 0; side < 2; ++side)
                for (int id : grouped.original_index(side == 0 ? i : j)) {
                    y.push_back(side == 0 ? +1 : -1);
                    dec_pair.push_back(dec_all[(size_t) id * n_binary_models + k]);
                }
            sigmoid_train(dec_pair, y, probA[k], probB[k]);
        }
}

// Labels from decision values (svc.cpp:265-316): one-vs-one vote, ties to the lowest class index; with
// probability estimates, the class of highest coupled probability (prob_predict keeps all of them).
std::vector<float_type> SVC::predict_label(const std::vector<float_type> &dec, int n_instances) {
    std::vector<float_type> out(n_instances);
    if (param.probability == 0) {
        std::vector<int> votes(n_classes);
        for (int r = 0; r < n_instances; ++r) {
            std::fill(votes.begin(), votes.end(), 0);
            int k = 0;
            for (int i = 0; i < n_classes; ++i)
                for (int j = i + 1; j < n_classes; ++j, ++k) votes[dec[(size_t) r * n_binary_models + k] > 0 ? i : j]++;
            int best = 0;
            for (int c = 1; c < n_classes; ++c) if (votes[c] > votes[best]) best = c;
            out[r] = (float) label[best];
        }
        return out;
    }
    TSVM_LOG << "predict with probability";
    prob_predict.clear();
    const float_type min_prob = 1e-7;
    std::vector<std::vector<float_type>> r(n_classes, std::vector<float_type>(n_classes));
    std::vector<float_type> p(n_classes);
    for (int row = 0; row < n_instances; ++row) {
        int k = 0;
        for (int i = 0; i < n_classes; ++i)
            for (int j = i + 1; j < n_classes; ++j, ++k) {
                r[i][j] = std::min(std::max(sigmoid_predict(dec[(size_t) row * n_binary_models + k], probA[k], probB[k]), min_prob),
                                   1 - min_prob);
                r[j][i] = 1 - r[i][j];
            }
        multiclass_probability(r, p);
        prob_predict.insert(prob_predict.end(), p.begin(), p.end());
        int best = 0;
        for (int c = 1; c < n_classes; ++c) if (p[c] > p[best]) best = c;
        out[row] = (float) label[best];
    }
    return out;
}

// ------------------------------------------------------------------------------------------------
// NuSVC (nusvc.cpp)
// ------------------------------------------------------------------------------------------------
void NuSVC::model_setup(const DataSet &dataset, SvmParam &p) {
    SVC::model_setup(dataset, p);
    param.svm_type = SvmParam::NU_SVC;
}

void NuSVC::setup_binary(const DataSet &dataset, int i, int j, BinaryProblem &p) {   // nusvc.cpp:17-50
    const std::vector<int> ids = dataset.original_index(i, j);
    const int n_pos = dataset.count()[i], n = (int) ids.size();
    p.i = i;
    p.j = j;
    p.y.resize(n);
    p.f_val.assign(n, 0);
    p.alpha.assign(n, 0);
    float_type sum_pos = param.nu * n / 2;
    float_type sum_neg = sum_pos;
    for (int l = 0; l < n; ++l) {
        float_type &budget = l < n_pos ? sum_pos : sum_neg;
        p.y[l] = l < n_pos ? +1 : -1;
        p.alpha[l] = std::min(1., budget);
        budget -= p.alpha[l];
    }
    p.k_mat.reset(new KernelMatrix(dataset, ids.data(), ids.size(), param));
    p.solver.reset(new NuSMOSolver(false));
    p.Cp = 1;
    p.Cn = 1;
}

// ------------------------------------------------------------------------------------------------
// SVR / NuSVR (svr.cpp, nusvr.cpp): the 2n-variable problem, instances stacked twice
// ------------------------------------------------------------------------------------------------
void SVR::model_setup(const DataSet &dataset, SvmParam &p) {
    n_classes = 2;
    SvmModel::model_setup(dataset, p);
    param.svm_type = SvmParam::EPSILON_SVR;
}

void SVR::train(const DataSet &dataset, SvmParam p) {
    model_setup(dataset, p);
    const int n = (int) dataset.n_instances();
    KernelMatrix k_mat(dataset, nullptr, n, param, 2);
    std::vector<float_type> f_val(2 * (size_t) n), alpha_2(2 * (size_t) n, 0);
    std::vector<int> y(2 * (size_t) n);
    for (int i = 0; i < n; ++i) {
        f_val[i] = param.p - dataset.y()[i];
        y[i] = +1;
        f_val[i + n] = -param.p - dataset.y()[i];
        y[i + n] = -1;
    }
    CSMOSolver solver;
    run_solver(solver, k_mat, y, alpha_2, rho[0], f_val, param.C, param.C);
    if (keep_binary) binary_alpha.push_back(alpha_2);
    save_svr_coef(alpha_2, dataset.instances());
    if (param.kernel_type == SvmParam::LINEAR) compute_linear_coef_single_model(dataset.n_features(), dataset.is_zero_based());
}

void SVR::save_svr_coef(const std::vector<float_type> &alpha_2, const DataSet::node2d &instances) {   // svr.cpp:43-62
    const size_t n = alpha_2.size() / 2;
    for (size_t i = 0; i < n; ++i) {
        const float_type a = alpha_2[i] - alpha_2[i + n];
        if (a != 0) {
            sv_indices.push_back((int) i);
            coef.push_back(a);
        }
    }
    copy_support_vectors(instances);
    n_sv[0] = (int) sv.size();
    n_sv[1] = 0;
    n_total_sv = (int) sv.size();
    TSVM_LOG << "rho = " << rho[0] << ", #sv = " << sv.size();
}

void NuSVR::model_setup(const DataSet &dataset, SvmParam &p) {
    SVR::model_setup(dataset, p);
    param.svm_type = SvmParam::NU_SVR;
}

void NuSVR::train(const DataSet &dataset, SvmParam p) {   // nusvr.cpp:7-41
    model_setup(dataset, p);
    const int n = (int) dataset.n_instances();
    KernelMatrix k_mat(dataset, nullptr, n, param, 2);
    std::vector<float_type> f_val(2 * (size_t) n), alpha_2(2 * (size_t) n);
    std::vector<int> y(2 * (size_t) n);
    float_type sum = param.C * param.nu * n / 2;
    for (int i = 0; i < n; ++i) {
        alpha_2[i] = alpha_2[i + n] = std::min(sum, param.C);
        sum -= alpha_2[i];
        f_val[i] = f_val[i + n] = -dataset.y()[i];
        y[i] = +1;
        y[i + n] = -1;
    }
    NuSMOSolver solver(true);
    run_solver(solver, k_mat, y, alpha_2, rho[0], f_val, param.C, param.C);
    if (keep_binary) binary_alpha.push_back(alpha_2);
    save_svr_coef(alpha_2, dataset.instances());
    if (param.kernel_type == SvmParam::LINEAR) compute_linear_coef_single_model(dataset.n_features(), dataset.is_zero_based());
}

// ------------------------------------------------------------------------------------------------
// OneClassSVC (oneclass_svc.cpp)
// ------------------------------------------------------------------------------------------------
void OneClassSVC::model_setup(const DataSet &dataset, SvmParam &p) {
    n_classes = 2;
    SvmModel::model_setup(dataset, p);
    param.svm_type = SvmParam::ONE_CLASS;
}

void OneClassSVC::train(const DataSet &dataset, SvmParam p) {
    model_setup(dataset, p);
    const int n = (int) dataset.n_instances();
    KernelMatrix k_mat(dataset, nullptr, n, param);
    std::vector<float_type> alpha(n, 0), f_val(n, 0);
    std::vector<int> y(n, 1);
    const int full = static_cast<int>(param.nu * n);
    for (int i = 0; i < full; ++i) alpha[i] = 1;
    if (full < n) alpha[full] = param.nu * n - full;
    CSMOSolver solver;
    run_solver(solver, k_mat, y, alpha, rho[0], f_val, 1, 1);
    if (keep_binary) binary_alpha.push_back(alpha);
    for (int i = 0; i < n; ++i)
        if (alpha[i] != 0) {
            sv_indices.push_back(i);
            coef.push_back(alpha[i]);
        }
    copy_support_vectors(dataset.instances());
    n_sv[0] = (int) sv.size();
    n_sv[1] = 0;
    n_total_sv = (int) sv.size();
    if (param.kernel_type == SvmParam::LINEAR) compute_linear_coef_single_model(dataset.n_features(), dataset.is_zero_based());
}

std::vector<float_type> OneClassSVC::finish_predict(int) {   // oneclass_svc.cpp:59-66
    std::vector<float_type> dec = dec_values;
    for (auto &v : dec) v = v > 0 ? 1 : -1;
    return dec;
}
