// Error reporting and version of the C ABI.
#include "../../include/thundersvm_amd.h"
#include "tsvm_internal.h"
#include <cstring>

static thread_local char g_err[512] = "";

void tsvm_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" {
const char *tsvm_last_error(void) { return g_err; }
int tsvm_version(void) { return 100; }
}
