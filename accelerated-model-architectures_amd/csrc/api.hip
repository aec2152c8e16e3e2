// Error slot and version query of the C ABI.
#include <stdarg.h>

#include "common.hpp"

namespace {
thread_local char g_error[512] = "";
}

void xma_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int xma_check_launch(const char *what) {
    hipError_t err = hipGetLastError();
    if (err == hipSuccess) return XMA_ROCM_OK;
    xma_set_error("%s: %s", what, hipGetErrorString(err));
    return XMA_ROCM_ELAUNCH;
}

extern "C" int xma_rocm_abi_version(void) { return XMA_ROCM_ABI_VERSION; }
extern "C" const char *xma_rocm_last_error(void) { return g_error; }
