// Error slot and version query of the C ABI.
#include <stdarg.h>

#include <mutex>
#include <set>
#include <utility>

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

int xma_set_max_lds_once(const void *kernel, int bytes) {
    static std::mutex lock;
    static std::set<std::pair<const void *, int>> done; // (kernel, device) pairs whose limit has been raised
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) {
        std::lock_guard<std::mutex> guard(lock);
        if (done.count({kernel, dev})) return XMA_ROCM_OK;
        err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (err == hipSuccess) {
            done.insert({kernel, dev});
            return XMA_ROCM_OK;
        }
    }
    xma_set_error("hipFuncSetAttribute(max dynamic LDS = %d): %s", bytes, hipGetErrorString(err));
    return XMA_ROCM_ELAUNCH;
}

extern "C" int xma_rocm_abi_version(void) { return XMA_ROCM_ABI_VERSION; }
extern "C" const char *xma_rocm_last_error(void) { return g_error; }
