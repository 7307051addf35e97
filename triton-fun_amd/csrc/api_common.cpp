// Version, thread-local last-error text and launch checking shared by all entry points.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "splat_common.hpp"

namespace splat {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return (int)e;
}

}  // namespace splat

extern "C" int splat_version(void) { return SPLAT_VERSION; }
extern "C" const char* splat_last_error(void) { return splat::g_err; }
