// thundersvm-predict: src/thundersvm/thundersvm-predict.cpp:18-106.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <fstream>

#include "cmdparser.h"
#include "models.h"

int main(int argc, char **argv) {
    CMDParser parser;
    try {
        parser.parse_predict(argc, argv, 1);
    } catch (const std::exception &e) {
        fprintf(stderr, "%s\n%s", e.what(), CMDParser::predict_usage());
        return 1;
    }
    try {
        tsvm::Log::enabled() = true;
        std::ifstream head(parser.svmpredict_model_file_name);
        if (!head.is_open()) {
            fprintf(stderr, "file %s not found\n", parser.svmpredict_model_file_name.c_str());
            return 1;
        }
        std::string key, type_name;
        head >> key >> type_name;
        if (key != "svm_type") throw std::runtime_error("model file does not start with svm_type");
        int type = -1;
        for (int i = 0; i < 5; ++i) if (type_name == SvmParam::svm_type_name[i]) type = i;
        if (type < 0) throw std::runtime_error("unknown svm_type in model file");
        std::unique_ptr<SvmModel> model = make_model((SvmParam::SVM_TYPE) type);
        TSVM_HIP_CHECK(hipSetDevice(parser.gpu_id));
        model->set_max_memory_size_Byte(parser.param_cmd.max_mem_size);
        auto now = [] { return std::chrono::high_resolution_clock::now(); };
        auto since = [&](std::chrono::high_resolution_clock::time_point t) { return std::chrono::duration<float>(now() - t).count(); };
        auto t0 = now();
        model->load_from_file(parser.svmpredict_model_file_name);
        TSVM_LOG << "model loading time = " << since(t0);
        DataSet test;
        t0 = now();
        test.load_from_file(parser.svmpredict_input_file);
        TSVM_LOG << "data loading time = " << since(t0);
        t0 = now();
        std::vector<float_type> predict_y = model->predict(test.instances(), -1);
        TSVM_LOG << "prediction time = " << since(t0);
        std::ofstream out(parser.svmpredict_output_file);
        for (float_type v : predict_y) out << v << '\n';   // (the reference ends each line with std::endl: the same bytes)
        if (type == SvmParam::C_SVC || type == SvmParam::NU_SVC)
            TSVM_LOG << "Accuracy = " << accuracy_score(predict_y, test.y());
        else if (type == SvmParam::EPSILON_SVR || type == SvmParam::NU_SVR)
            TSVM_LOG << "Mean Squared Error = " << mse_score(predict_y, test.y());
    } catch (std::bad_alloc &) {
        fprintf(stderr, "out of memory, you may try \"-m memory size\" to constrain memory usage\n");
        return EXIT_FAILURE;
    } catch (const std::exception &e) {
        fprintf(stderr, "%s\n", e.what());
        return EXIT_FAILURE;
    }
    return 0;
}
