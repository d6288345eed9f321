// Host-side helpers shared by every C-ABI entry point: status codes, the thread-local
// error message, and launch checking.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/comp_inference_hip.h"

namespace ci {

extern thread_local char g_err[512];

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

inline int hip_fail(hipError_t e, const char *what) {
    return fail(CI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define CI_HIP(call)                                         \
    do {                                                     \
        hipError_t e_ = (call);                              \
        if (e_ != hipSuccess) return ci::hip_fail(e_, #call); \
    } while (0)

// A kernel launch reports configuration errors through hipGetLastError only.
#define CI_LAUNCH_CHECK(name)                                  \
    do {                                                       \
        hipError_t e_ = hipGetLastError();                     \
        if (e_ != hipSuccess) return ci::hip_fail(e_, name);   \
    } while (0)

inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Largest LDS allocation a workgroup may ask for on gfx950 (160 KB per CU).
constexpr uint32_t kLdsLimit = 160 * 1024;

}  // namespace ci
