// Host-side helpers shared by every C-ABI entry point: status codes, the thread-local
// error message, and launch checking.  gfx950 only.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
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

// How the streams of a tile lie in the byte stream, for the kernels that take every layout.
//   kBodyTwo   two streams per column (rows [0, th/2) and [th/2, th)), tile body of 2 tw bytes a row (default)
//   kExactBytes one stream per column over the tile's height, each stream's bytes on their own at stream_offsets
//   kBodyOne   one stream per column over the tile's height, tile body of tw bytes a row
enum TileLayout { kBodyTwo = 0, kExactBytes = 1, kBodyOne = 2 };

inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Largest LDS allocation a workgroup may ask for on gfx950 (160 KB per CU).
constexpr uint32_t kLdsLimit = 160 * 1024;

// CUs of the current device.
inline int cu_count(uint32_t *out) {
    int dev = 0, n = 0;
    CI_HIP(hipGetDevice(&dev));
    CI_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
    *out = n > 0 ? (uint32_t)n : 1u;
    return CI_OK;
}

// Lets kernel `fn` ask for the whole LDS.  The attribute belongs to (function, device): `done` is the
// call site's record of the devices it has been set on (bit = device index), safe to share between
// threads -- two threads setting it at once set the same value.
inline int allow_full_lds(const void *fn, std::atomic<uint64_t> &done) {
    int dev = 0;
    CI_HIP(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return CI_OK;
    CI_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
    done.fetch_or(bit, std::memory_order_release);
    return CI_OK;
}
#define CI_ALLOW_FULL_LDS(kernel)                                                             \
    do {                                                                                      \
        static std::atomic<uint64_t> done_{0};                                                \
        if (int rc_ = ci::allow_full_lds(reinterpret_cast<const void *>(kernel), done_)) return rc_; \
    } while (0)

}  // namespace ci
