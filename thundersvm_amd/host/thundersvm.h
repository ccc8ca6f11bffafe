// Basic types of the host layer.  float_type and kernel_type are both double: the reference built
// with -DUSE_DOUBLE=ON (include/thundersvm/thundersvm.h:16-22).
#pragma once
#include <cstddef>
#include <cstdint>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

typedef double float_type;
typedef double kernel_type;

namespace tsvm {
// Tiny logger standing in for the reference's easylogging++ LOG(INFO); silenced by `-q`
// (src/thundersvm/cmdparser.cpp:210).
struct Log {
    static bool &enabled() { static bool e = false; return e; }
    std::ostringstream os;
    ~Log() { if (enabled()) std::cerr << os.str() << std::endl; }
};
}  // namespace tsvm
#define TSVM_LOG ::tsvm::Log().os
