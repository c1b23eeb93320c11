// Error reporting shared by the C entry points: the last message per thread, in the
// manner of a C library that returns int status codes (tq-kv/src/ffi.rs:89-108).
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include "tq_kernels.h"

static thread_local char g_last_error[512] = "";

int tqk_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return -1;
}

int tqk_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    return tqk_fail("%s: launch failed: %s", what, hipGetErrorString(e));
}

extern "C" const char* tqk_last_error(void) { return g_last_error; }
extern "C" int tqk_abi_version(void) { return 13; }
