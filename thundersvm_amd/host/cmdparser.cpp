#include "cmdparser.h"

#include <omp.h>

#include <cstdlib>
#include <cstring>

const char *CMDParser::train_usage() {
    return "Usage: thundersvm-train [options] training_set_file [model_file]\n"
           "options:\n"
           "-s svm_type: 0 C-SVC, 1 nu-SVC, 2 one-class SVM, 3 epsilon-SVR, 4 nu-SVR (default 0)\n"
           "-t kernel_type: 0 linear, 1 polynomial, 2 radial basis function, 3 sigmoid (default 2)\n"
           "-d degree (default 3)   -g gamma (default 1/num_features)   -r coef0 (default 0)\n"
           "-c cost (default 1)   -n nu (default 0.5)   -p epsilon of epsilon-SVR (default 0.1)\n"
           "-m memory size in MB (default 8192)   -e tolerance of termination criterion (default 0.001)\n"
           "-b probability_estimates: 0 or 1 (C-SVC, nu-SVC)   -wi weight: C of class i = weight*C\n"
           "-v n: n-fold cross validation   -u n: gpu to use (default 0)   -o n: cpu cores (-1 = all)   -q quiet\n";
}

const char *CMDParser::predict_usage() {
    return "Usage: thundersvm-predict [options] test_file model_file output_file\n"
           "options:\n-m memory size in MB (default 8192)   -u n: gpu to use (default 0)   -o n: cpu cores\n";
}

static float_type parse_gamma(const char *s) {   // "1/8" style fractions are accepted
    const char *slash = strchr(s, '/');
    if (!slash) return atof(s);
    return atof(std::string(s, slash).c_str()) / atof(slash + 1);
}

void CMDParser::parse_command_line(int argc, char **argv) {
    std::string bin = argv[0];
    bin = bin.substr(bin.find_last_of("/\\") + 1);
    if (bin.rfind("thundersvm-predict", 0) == 0) parse_predict(argc, argv, 1);
    else parse_train(argc, argv, 1);
}

void CMDParser::parse_train(int argc, char **argv, int first) {
    int i = first;
    for (; i < argc && argv[i][0] == '-'; ++i) {
        const char opt = argv[i][1];
        if (opt == 'q') { quiet = true; continue; }
        if (i + 1 >= argc) throw std::invalid_argument(std::string("option needs a value: ") + argv[i]);
        const char *flag = argv[i];
        const char *val = argv[++i];
        switch (opt) {
            case 's': param_cmd.svm_type = static_cast<SvmParam::SVM_TYPE>(atoi(val)); break;
            case 't': param_cmd.kernel_type = static_cast<SvmParam::KERNEL_TYPE>(atoi(val)); break;
            case 'd': param_cmd.degree = atoi(val); break;
            case 'g': param_cmd.gamma = parse_gamma(val); gamma_set = true; break;
            case 'r': param_cmd.coef0 = atof(val); break;
            case 'n': param_cmd.nu = atof(val); break;
            case 'm': param_cmd.max_mem_size = static_cast<size_t>(std::max(atoi(val), 0)) << 20; break;
            case 'c': param_cmd.C = atof(val); break;
            case 'e': param_cmd.epsilon = atof(val); break;
            case 'p': param_cmd.p = atof(val); break;
            case 'h': break;   // shrinking: accepted and ignored, as in the reference
            case 'b': param_cmd.probability = atoi(val); break;
            case 'o': n_cores = atoi(val); break;
            case 'u': gpu_id = atoi(val); break;
            case 'v':
                do_cross_validation = true;
                nr_fold = atoi(val);
                if (nr_fold < 2) throw std::invalid_argument("n-fold cross validation: n must >= 2");
                break;
            case 'w':
                weight_labels_.push_back(atoi(flag + 2));
                weights_.push_back(atof(val));
                break;
            default: throw std::invalid_argument(std::string("Unknown option: ") + flag);
        }
    }
    param_cmd.nr_weight = (int) weights_.size();
    param_cmd.weight_label = weight_labels_.empty() ? nullptr : weight_labels_.data();
    param_cmd.weight = weights_.empty() ? nullptr : weights_.data();
    if (n_cores > 0) omp_set_num_threads(n_cores);
    else if (n_cores != -1) throw std::invalid_argument("the number of cpu cores must be positive or -1");
    if (i >= argc) throw std::invalid_argument("no training file given");
    if (!check_parameter()) throw std::invalid_argument("invalid parameter");
    svmtrain_input_file_name = argv[i];
    if (i + 1 < argc) {
        model_file_name = argv[i + 1];
    } else {
        const std::string in = argv[i];
        model_file_name = in.substr(in.find_last_of('/') + 1) + ".model";
    }
}

void CMDParser::parse_predict(int argc, char **argv, int first) {
    int i = first;
    for (; i < argc && argv[i][0] == '-'; ++i) {
        const char opt = argv[i][1];
        if (i + 1 >= argc) throw std::invalid_argument(std::string("option needs a value: ") + argv[i]);
        const char *val = argv[++i];
        switch (opt) {
            case 'b': break;
            case 'u': gpu_id = atoi(val); break;
            case 'o': n_cores = atoi(val); break;
            case 'm': param_cmd.max_mem_size = static_cast<size_t>(std::max(atoi(val), 0)) << 20; break;
            default: throw std::invalid_argument(std::string("Unknown option: -") + opt);
        }
    }
    if (n_cores > 0) omp_set_num_threads(n_cores);
    if (i + 2 >= argc) throw std::invalid_argument("expected: test_file model_file output_file");
    svmpredict_input_file = argv[i];
    svmpredict_model_file_name = argv[i + 1];
    svmpredict_output_file = argv[i + 2];
}

bool CMDParser::check_parameter() const {   // cmdparser.cpp:303-355
    const SvmParam &p = param_cmd;
    if (p.svm_type < SvmParam::C_SVC || p.svm_type > SvmParam::NU_SVR) return false;
    if (p.kernel_type < SvmParam::LINEAR || p.kernel_type > SvmParam::PRECOMPUTED) return false;
    if (p.gamma < 0 || p.degree < 0 || p.epsilon <= 0) return false;
    const bool uses_c = p.svm_type == SvmParam::C_SVC || p.svm_type == SvmParam::EPSILON_SVR || p.svm_type == SvmParam::NU_SVR;
    if (uses_c && p.C <= 0) return false;
    const bool uses_nu = p.svm_type == SvmParam::NU_SVC || p.svm_type == SvmParam::ONE_CLASS || p.svm_type == SvmParam::NU_SVR;
    if (uses_nu && (p.nu <= 0 || p.nu > 1)) return false;
    if (p.svm_type == SvmParam::EPSILON_SVR && p.p < 0) return false;
    if (p.max_mem_size <= 0) return false;
    if (p.probability != 0 && p.probability != 1) return false;
    if (p.probability == 1 && !(p.svm_type == SvmParam::C_SVC || p.svm_type == SvmParam::NU_SVC)) return false;
    return true;
}

float_type accuracy_score(const std::vector<float_type> &predict_y, const std::vector<float_type> &truth) {
    int correct = 0;
    for (size_t i = 0; i < predict_y.size(); ++i) correct += predict_y[i] == truth[i];
    return correct / (float) truth.size();
}

float_type mse_score(const std::vector<float_type> &predict_y, const std::vector<float_type> &truth) {
    float_type s = 0;
    for (size_t i = 0; i < predict_y.size(); ++i) s += (predict_y[i] - truth[i]) * (predict_y[i] - truth[i]);
    return s / predict_y.size();
}
