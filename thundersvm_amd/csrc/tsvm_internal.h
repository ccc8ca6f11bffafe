// Host-side plumbing shared by the C ABI translation units: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>

void tsvm_set_error(const char *fmt, ...);

#define TSVM_REQUIRE(cond, ...)                \
    do {                                       \
        if (!(cond)) {                         \
            tsvm_set_error(__VA_ARGS__);       \
            return -1; /* TSVM_EINVAL */       \
        }                                      \
    } while (0)

#define TSVM_HIP(expr)                                                                   \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess) {                                                          \
            tsvm_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return (int) e_;                                                             \
        }                                                                                \
    } while (0)

#define TSVM_LAUNCH_CHECK() TSVM_HIP(hipGetLastError())

static inline hipStream_t tsvm_s(void *s) { return (hipStream_t) s; }
