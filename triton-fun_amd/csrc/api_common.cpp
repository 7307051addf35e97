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

// An error left behind by another user of the runtime on this thread stays pending until someone reads it.  It must not
// be taken for a failure of this library's launch, and it must not vanish either (its owner may not have looked yet):
// it is read away before launching, remembered, and handed to the caller by check_launch() under its own name.
static thread_local hipError_t g_foreign = hipSuccess;

void begin_launch() {
    if (hipPeekAtLastError() != hipSuccess) g_foreign = hipGetLastError();
}

int check_launch(const char* what) {
    const hipError_t foreign = g_foreign;
    g_foreign = hipSuccess;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return (int)e;
    }
    if (foreign != hipSuccess) {
        set_error("%s: a runtime error from an earlier call on this thread was still pending when this call began (%s); "
                  "this call's own launch went through",
                  what, hipGetErrorString(foreign));
        return (int)foreign;
    }
    return 0;
}

int reserve_dynamic_lds(uint64_t* done, const void* kernel, size_t bytes, const char* who) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        set_error("%s: hipGetDevice: %s", who, hipGetErrorString(e));
        return (int)e;
    }
    const uint64_t bit = 1ull << (dev & 63);
    if (__atomic_load_n(done, __ATOMIC_ACQUIRE) & bit) return 0;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
        set_error("%s: cannot reserve %zu bytes of LDS: %s", who, bytes, hipGetErrorString(e));
        return (int)e;
    }
    __atomic_fetch_or(done, bit, __ATOMIC_RELEASE);
    return 0;
}

}  // namespace splat

extern "C" int splat_version(void) { return SPLAT_VERSION; }
extern "C" const char* splat_last_error(void) { return splat::g_err; }
