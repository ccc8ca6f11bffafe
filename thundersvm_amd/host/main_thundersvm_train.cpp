// thundersvm-train: same options, default model-file name and "all training time" window as
// src/thundersvm/thundersvm-train.cpp:21-136.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>

#include "cmdparser.h"
#include "models.h"

int main(int argc, char **argv) {
    CMDParser parser;
    try {
        parser.parse_train(argc, argv, 1);
    } catch (const std::exception &e) {
        fprintf(stderr, "%s\n%s", e.what(), CMDParser::train_usage());
        return 1;
    }
    // A process that trains once and exits pays for the row arena's allocation and release once per training: the
    // release alone takes 0.5 s for three quarters of the device's memory and 1.8 s for nine tenths, and the driver clears
    // released memory in the background (about 40 GB/s) before it hands it out again, so a process that asks for more
    // than the untouched rest right after another has exited waits for that (two such runs with half of the memory
    // each: the second trains in 5.8 s instead of 1.75 s).  The library's default (nine tenths of the free memory) suits
    // processes that train again and again; here less than half is taken unless the environment says otherwise, so that
    // one run after another finds an untouched half.
    setenv("TSVM_ARENA_PERCENT", "45", 0);
    try {
        tsvm::Log::enabled() = !parser.quiet;
        DataSet train;
        auto t_load = std::chrono::high_resolution_clock::now();
        train.load_from_file(parser.svmtrain_input_file_name);
        TSVM_LOG << "data loading time = " << std::chrono::duration<float>(std::chrono::high_resolution_clock::now() - t_load).count();
        std::unique_ptr<SvmModel> model = make_model(parser.param_cmd.svm_type);
        if (parser.param_cmd.svm_type == SvmParam::NU_SVC) {   // feasibility of nu (thundersvm-train.cpp:57-70)
            train.group_classes();
            for (size_t i = 0; i < train.n_classes(); ++i)
                for (size_t j = i + 1; j < train.n_classes(); ++j) {
                    const int n1 = train.count()[i], n2 = train.count()[j];
                    if (parser.param_cmd.nu * (n1 + n2) / 2 > std::min(n1, n2)) {
                        printf("specified nu is infeasible\n");
                        return 1;
                    }
                }
        }
        if (parser.param_cmd.kernel_type != SvmParam::LINEAR && !parser.gamma_set) {
            parser.param_cmd.gamma = 1.f / train.n_features();
            TSVM_LOG << "using default gamma=" << parser.param_cmd.gamma;
        }
        TSVM_HIP_CHECK(hipSetDevice(parser.gpu_id));
        if (parser.do_cross_validation) {
            std::vector<float_type> predict_y = model->cross_validation(train, parser.param_cmd, parser.nr_fold);
            const SvmParam::SVM_TYPE t = parser.param_cmd.svm_type;
            if (t == SvmParam::C_SVC || t == SvmParam::NU_SVC)
                std::cout << "Cross Accuracy = " << accuracy_score(predict_y, train.y()) << std::endl;
            else if (t == SvmParam::EPSILON_SVR || t == SvmParam::NU_SVR)
                std::cout << "Cross Mean Squared Error = " << mse_score(predict_y, train.y()) << std::endl;
        } else {
            auto start = std::chrono::high_resolution_clock::now();
            model->train(train, parser.param_cmd);
            std::chrono::duration<float> dt = std::chrono::high_resolution_clock::now() - start;
            TSVM_LOG << "all training time = " << dt.count();
            auto t_save = std::chrono::high_resolution_clock::now();
            model->save_to_file(parser.model_file_name);
            TSVM_LOG << "model saving time = " << std::chrono::duration<float>(std::chrono::high_resolution_clock::now() - t_save).count();
        }
    } catch (std::bad_alloc &) {
        fprintf(stderr, "out of memory, you may try \"-m memory size\" to constrain memory usage\n");
        return EXIT_FAILURE;
    } catch (const std::exception &e) {
        fprintf(stderr, "%s\n", e.what());
        return EXIT_FAILURE;
    }
    return 0;
}
