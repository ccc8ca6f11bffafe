// SvmModel and its five concrete models (SVC, NuSVC, OneClassSVC, SVR, NuSVR): problem set-up,
// one-vs-one decomposition, LibSVM coefficient layout, prediction and the LibSVM-compatible model
// file.  Public surface of include/thundersvm/model/{svmmodel,svc,nusvc,oneclass_svc,svr,nusvr}.h;
// kernel evaluation and the SMO solve run on the GPU through KernelMatrix / CSMOSolver.
#pragma once
#include <memory>

#include "dataset.h"
#include "kernelmatrix.h"
#include "solver.h"
#include "svmparam.h"

class SvmModel {
public:
    virtual ~SvmModel() = default;
    virtual void train(const DataSet &dataset, SvmParam param) = 0;
    std::vector<float_type> predict(const DataSet::node2d &instances, int batch_size = -1);
    void predict_dec_values(const DataSet::node2d &instances, std::vector<float_type> &dec_values, int batch_size) const;
    // The same for the instances of a DataSet; when the DataSet has a device-resident copy of its rows in the dense
    // layout (DeviceRows::of), the kernels read the rows where they lie: nothing is assembled on the host or uploaded.
    std::vector<float_type> predict(const DataSet &dataset, int batch_size = -1);
    void predict_dec_values(const DataSet &dataset, std::vector<float_type> &dec_values, int batch_size) const;
    virtual std::vector<float_type> cross_validation(DataSet dataset, SvmParam param, int n_fold);

    virtual void save_to_file(std::string path);
    virtual std::string save_to_string();
    virtual void load_from_file(std::string path);
    virtual void load_from_string(std::string data);

    int total_sv() const { return n_total_sv; }
    const DataSet::node2d &svs() const { return sv; }
    const std::vector<int> &get_n_sv() const { return n_sv; }
    const std::vector<float_type> &get_coef() const { return coef; }
    const std::vector<float_type> &get_linear_coef() const { return linear_coef; }
    const std::vector<float_type> &get_rho() const { return rho; }
    int get_n_classes() const { return n_classes; }
    int get_sv_max_index() const { return sv_max_index; }
    const std::vector<int> &get_sv_ind() const { return sv_indices; }
    const std::vector<int> &get_label() const { return label; }
    void set_max_iter(int iter) { max_iter = iter; }
    void set_max_memory_size(size_t size_mb) { if (size_mb > 0) param.max_mem_size = size_mb << 20; }
    void set_max_memory_size_Byte(size_t size) { if (size > 0) param.max_mem_size = size; }
    const std::vector<float_type> &get_dec_value() const { return dec_values; }
    int get_n_binary_models() const { return n_binary_models; }
    const std::vector<float> &get_prob_predict() const { return prob_predict; }
    bool is_prob() const { return param.probability; }
    const SvmParam &get_param() const { return param; }
    int get_working_set_size(const KernelMatrix &k_mat, size_t held_bytes = 0);

    // diagnostics of the last train() call, one entry per binary sub-problem
    std::vector<SolverStats> solver_stats;
    std::vector<std::vector<float_type>> binary_alpha;   // signed alpha (alpha*y), training order of the sub-problem
    std::vector<std::vector<float_type>> binary_f;
    SolverTrace *trace_first = nullptr;   // when set, the first sub-problem records its trajectory here
    int ws_override = 0;                  // > 0 forces the working-set size
    bool profile = false;
    bool keep_binary = false;             // keep binary_alpha / binary_f (tests)
    long long cache_bytes = -1;           // kernel-row cache budget handed to the solver (-1 auto, 0 off)
    int pair_lanes = 0;                   // class pairs of a one-vs-one run in flight (0: automatic, 1: one at a time)

protected:
    virtual void model_setup(const DataSet &dataset, SvmParam &param);
    // what predict returns once dec_values holds the decision values of n_instances rows: the values themselves,
    // class labels (SVC) or the side of the boundary (OneClassSVC)
    virtual std::vector<float_type> finish_predict(int n_instances) { return dec_values; }
    // the model as the prediction kernels read it (support vectors in HBM, coefficients by padded column)
    struct PredictPlan;
    const PredictPlan &predict_plan() const;
    // one batch, rows already on the device as a dense matrix; false when the kernels do not take this model's shape
    bool predict_batch_fused(const PredictPlan &plan, const kernel_type *a, int64_t lda, const kernel_type *sd_a, size_t m,
                             bool indicator_values, float_type *dec_out) const;
    void copy_support_vectors(const DataSet::node2d &instances);
    void run_solver(CSMOSolver &solver, const KernelMatrix &k_mat, const std::vector<int> &y, std::vector<float_type> &alpha,
                    float_type &rho, std::vector<float_type> &f_val, float_type Cp, float_type Cn, size_t held_bytes = 0);
    void compute_linear_coef_single_model(size_t n_feature, bool zero_based);

    SvmParam param;
    std::vector<int> own_weight_label;        // what param.weight_label / param.weight point at
    std::vector<float_type> own_weight;
    std::vector<float_type> coef;
    std::vector<float_type> linear_coef;
    DataSet::node2d sv;
    mutable std::shared_ptr<KernelMatrix> sv_k_mat;   // device copy of sv, built by the first predict call
    mutable std::shared_ptr<PredictPlan> predict_plan_;
    std::vector<int> sv_indices;
    std::vector<int> n_sv;           // per class
    int n_total_sv = 0;
    std::vector<float_type> rho;
    int n_classes = 2;
    int n_binary_models = 1;
    int max_iter = -1;
    std::vector<float_type> dec_values;
    std::vector<int> label;
    std::vector<float_type> probA, probB;
    std::vector<float> prob_predict;
    int sv_max_index = 0;
};

class SVC : public SvmModel {
public:
    void train(const DataSet &dataset, SvmParam param) override;

protected:
    void model_setup(const DataSet &dataset, SvmParam &param) override;
    std::vector<float_type> finish_predict(int n_instances) override;
    // One class pair (i, j) of the one-vs-one decomposition: its rows, labels, starting point and solver.
    struct BinaryProblem {
        int i = 0, j = 0, k = 0;
        std::unique_ptr<KernelMatrix> k_mat;
        std::unique_ptr<CSMOSolver> solver;
        std::vector<int> y;
        std::vector<float_type> alpha, f_val;
        float_type Cp = 0, Cn = 0;
        // lockstep execution
        std::unique_ptr<SolveTask> task;
        hipEvent_t rows_done = nullptr, solved = nullptr;
        int lane = 0;
        bool rows_pending = false;   // independent lanes: the iteration's rows and update_f are still to be enqueued
    };
    virtual void setup_binary(const DataSet &dataset, int i, int j, BinaryProblem &p);   // svc.cpp:147-170
    void finish_binary(BinaryProblem &p, std::vector<float_type> &alpha_out);            // svc.cpp:171-177
    void train_pairs_in_lockstep(const DataSet &grouped, int lanes, std::vector<std::vector<float_type>> &alpha);
    std::vector<float_type> predict_label(const std::vector<float_type> &dec_values, int n_instances);
    void probability_train(const DataSet &grouped);                                            // svc.cpp:432-491
    void multiclass_probability(const std::vector<std::vector<float_type>> &r, std::vector<float_type> &p) const;   // svc.cpp:206-263
    std::vector<float_type> c_weight;
};

class NuSVC : public SVC {
protected:
    void model_setup(const DataSet &dataset, SvmParam &param) override;
    void setup_binary(const DataSet &dataset, int i, int j, BinaryProblem &p) override;
};

class SVR : public SvmModel {
public:
    void train(const DataSet &dataset, SvmParam param) override;

protected:
    void model_setup(const DataSet &dataset, SvmParam &param) override;
    void save_svr_coef(const std::vector<float_type> &alpha_2, const DataSet::node2d &instances);
};

class NuSVR : public SVR {
public:
    void train(const DataSet &dataset, SvmParam param) override;

protected:
    void model_setup(const DataSet &dataset, SvmParam &param) override;
};

class OneClassSVC : public SvmModel {
public:
    void train(const DataSet &dataset, SvmParam param) override;

protected:
    void model_setup(const DataSet &dataset, SvmParam &param) override;
    std::vector<float_type> finish_predict(int n_instances) override;
};

// Factory keyed on SvmParam::SVM_TYPE (thundersvm-train.cpp:41-60).
std::unique_ptr<SvmModel> make_model(SvmParam::SVM_TYPE type);
