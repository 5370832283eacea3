// Error plumbing and ABI version of liblatentq_hip.so.
#include "lq_common.h"

#include <atomic>
#include <stdarg.h>
#include <stdio.h>

namespace {
thread_local char g_err[512] = "";
}

int lq_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int lq_check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return lq_fail(LQ_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return LQ_OK;
}

// Compute units of the current device. The only state the library keeps between calls besides the
// per-thread error text: one relaxed atomic per device ordinal, written with the value the runtime
// reports (every thread that races here writes the same number).
int lq_device_cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

extern "C" int lq_abi_version(void) { return 2; }

extern "C" const char *lq_last_error(void) { return g_err; }
