// SvmParam: same fields and defaults as include/thundersvm/svmparam.h:14-66.
#pragma once
#include "thundersvm.h"

struct SvmParam {
    enum SVM_TYPE { C_SVC, NU_SVC, ONE_CLASS, EPSILON_SVR, NU_SVR };
    enum KERNEL_TYPE { LINEAR, POLY, RBF, SIGMOID, PRECOMPUTED };

    SVM_TYPE svm_type = C_SVC;
    KERNEL_TYPE kernel_type = RBF;
    float_type C = 1;
    float_type gamma = 0;
    float_type p = 0.1f;          // float literals in the reference: 0.1f, 0.001f
    float_type nu = 0.5;
    float_type epsilon = 0.001f;
    int degree = 3;
    float_type coef0 = 0;
    int nr_weight = 0;
    int *weight_label = nullptr;
    float_type *weight = nullptr;
    int probability = 0;
    size_t max_mem_size = static_cast<size_t>(8192) << 20;

    static const char *kernel_type_name[6];
    static const char *svm_type_name[6];
};
