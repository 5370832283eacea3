// Error plumbing and ABI version of liblatentq_hip.so.
#include "lq_common.h"

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

extern "C" int lq_abi_version(void) { return 1; }

extern "C" const char *lq_last_error(void) { return g_err; }
