// CMDParser: the LibSVM-compatible command line of thundersvm-train / thundersvm-predict
// (flags of src/thundersvm/cmdparser.cpp:59-211: -s -t -d -g -r -c -n -p -m -e -b -w<label> -v -u -o -q).
// Invalid values throw std::invalid_argument instead of printing the help text and exiting, so the
// library stays usable from tests; the executables print the usage and exit with status 1.
#pragma once
#include <stdexcept>

#include "svmparam.h"

class CMDParser {
public:
    void parse_command_line(int argc, char **argv);   // argv[0] decides train vs predict, as in the reference
    void parse_train(int argc, char **argv, int first);
    void parse_predict(int argc, char **argv, int first);
    bool check_parameter() const;
    static const char *train_usage();
    static const char *predict_usage();

    SvmParam param_cmd;
    bool do_cross_validation = false;
    bool gamma_set = false;
    bool quiet = false;
    int nr_fold = 0;
    int gpu_id = 0;
    int n_cores = -1;
    std::string svmtrain_input_file_name, model_file_name;
    std::string svmpredict_input_file, svmpredict_output_file, svmpredict_model_file_name;

private:
    std::vector<int> weight_labels_;
    std::vector<float_type> weights_;
};

// Accuracy / MSE (src/thundersvm/util/metric.cpp:10-31)
float_type accuracy_score(const std::vector<float_type> &predict_y, const std::vector<float_type> &truth);
float_type mse_score(const std::vector<float_type> &predict_y, const std::vector<float_type> &truth);
