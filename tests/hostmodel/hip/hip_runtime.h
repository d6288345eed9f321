// Stand-in for <hip/hip_runtime.h> when the library's HIP sources are compiled for the host model
// (tests/hostmodel/sim.h): the kernels then run on the CPU, one fibre per thread of a workgroup, with every
// wavefront-wide operation, barrier, matrix instruction and hand-written assembly statement carried out by the
// model.  Test infrastructure: nothing of the product includes this file.
#pragma once
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#include "../sim.h"

#define __host__
#define __device__
#define __global__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
// (__shared__ is left alone: the build rewrites those declarations after preprocessing)

// ---- vector types the sources use --------------------------------------------------------------------------
struct uint2 {
    uint32_t x, y;
};
struct uint4 {
    uint32_t x, y, z, w;
};
struct float4 {
    float x, y, z, w;
};
static inline uint2 make_uint2(uint32_t x, uint32_t y) { return uint2{x, y}; }
static inline uint4 make_uint4(uint32_t x, uint32_t y, uint32_t z, uint32_t w) { return uint4{x, y, z, w}; }
static inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
typedef sim::Dim3 dim3;

#define threadIdx (sim::lane_ctx().thread_idx)
#define blockIdx (sim::lane_ctx().block_idx)
#define blockDim (sim::lane_ctx().block_dim)
#define gridDim (sim::lane_ctx().grid_dim)

// ---- device functions ---------------------------------------------------------------------------------------
static inline uint32_t __umul24(uint32_t a, uint32_t b) { return (a & 0xFFFFFFu) * (b & 0xFFFFFFu); }
static inline uint32_t __float_as_uint(float f) { return __builtin_bit_cast(uint32_t, f); }
static inline int __float_as_int(float f) { return __builtin_bit_cast(int, f); }
static inline float __uint_as_float(uint32_t u) { return __builtin_bit_cast(float, u); }
static inline float __int_as_float(int u) { return __builtin_bit_cast(float, u); }
static inline int __popc(uint32_t v) { return __builtin_popcount(v); }
static inline int __popcll(uint64_t v) { return __builtin_popcountll(v); }
static inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
static inline int __clz(int v) { return v ? __builtin_clz((uint32_t)v) : 32; }

#define CI_SIM_MINMAX(T)                                   \
    static inline T min(T a, T b) { return b < a ? b : a; } \
    static inline T max(T a, T b) { return a < b ? b : a; }
CI_SIM_MINMAX(int)
CI_SIM_MINMAX(unsigned)
CI_SIM_MINMAX(long)
CI_SIM_MINMAX(unsigned long)
CI_SIM_MINMAX(long long)
CI_SIM_MINMAX(unsigned long long)
CI_SIM_MINMAX(float)
CI_SIM_MINMAX(double)
#undef CI_SIM_MINMAX

#define __syncthreads() sim::syncthreads()
#define __builtin_amdgcn_ballot_w64(p) sim::ballot((p) ? 1 : 0)
#define __builtin_amdgcn_readlane(v, l) sim::readlane((int)(v), (int)(l))
#define __builtin_amdgcn_readfirstlane(v) sim::readfirstlane((int)(v))
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) sim::update_dpp((int)(old), (int)(src), (ctrl), (rm), (bm), (bc))
#define __builtin_amdgcn_permlane16_swap(a, b, fi, bc) sim::permlane_swap((uint32_t)(a), (uint32_t)(b), 16)
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) sim::permlane_swap((uint32_t)(a), (uint32_t)(b), 32)
#define __builtin_amdgcn_perm(a, b, sel) sim::v_perm((uint32_t)(a), (uint32_t)(b), (uint32_t)(sel))
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define __builtin_amdgcn_wave_barrier() sim::wave_sync()
#define __builtin_amdgcn_s_sleep(n) sim::yield()
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) sim::mfma_32x32x16_bf16((a), (b), (c))
#define __shfl(v, src, width) sim::shfl((int)(v), (int)(src), (int)(width))
#define __shfl_up(v, d, width) sim::shfl_up((int)(v), (unsigned)(d), (int)(width))

// One thread runs at a time: plain reads and writes are atomic.  In the build that checks the ordering between
// wavefronts these functions are not instrumented: an atomic access is told to the model as such (sim::order_atomic).
#define CI_SIM_ATOMIC_FN __attribute__((no_sanitize("thread"))) static inline
template <typename T>
CI_SIM_ATOMIC_FN T atomicAdd(T *p, T v) {
    sim::order_atomic(p, true, true);
    T o = *p;
    *p = o + v;
    return o;
}
template <typename T>
CI_SIM_ATOMIC_FN T atomicMax(T *p, T v) {
    sim::order_atomic(p, true, true);
    T o = *p;
    if (v > o) *p = v;
    return o;
}
template <typename T>
CI_SIM_ATOMIC_FN T atomicOr(T *p, T v) {
    sim::order_atomic(p, true, true);
    T o = *p;
    *p = o | v;
    return o;
}
#define __HIP_MEMORY_SCOPE_WORKGROUP 0
// (an operation that publishes -- release semantics -- comes after what the other lanes of the wavefront did earlier
// in the program: sim::wave_catch_up)
#define CI_SIM_RELEASES(order) ((order) == __ATOMIC_RELEASE || (order) == __ATOMIC_ACQ_REL || (order) == __ATOMIC_SEQ_CST)
#define CI_SIM_ACQUIRES(order) ((order) == __ATOMIC_ACQUIRE || (order) == __ATOMIC_ACQ_REL || (order) == __ATOMIC_SEQ_CST)
template <typename T>
CI_SIM_ATOMIC_FN T ci_sim_atomic_load(T *p, int order) {
    const T v = *(volatile T *)p;
    sim::order_atomic(p, CI_SIM_ACQUIRES(order), false);
    return v;
}
template <typename T, typename V>
CI_SIM_ATOMIC_FN void ci_sim_atomic_store(T *p, V v, int order) {
    if (CI_SIM_RELEASES(order)) sim::wave_catch_up();
    sim::order_atomic(p, false, CI_SIM_RELEASES(order));
    *(volatile T *)p = (T)v;
}
template <typename T, typename V>
CI_SIM_ATOMIC_FN T ci_sim_atomic_fetch_add(T *p, V v, int order) {
    if (CI_SIM_RELEASES(order)) sim::wave_catch_up();
    sim::order_atomic(p, CI_SIM_ACQUIRES(order), CI_SIM_RELEASES(order));
    const T o = *(volatile T *)p;
    *(volatile T *)p = o + (T)v;
    return o;
}
#define __hip_atomic_load(p, order, scope) ci_sim_atomic_load((p), (order))
#define __hip_atomic_store(p, v, order, scope) ci_sim_atomic_store((p), (v), (order))
#define __hip_atomic_fetch_add(p, v, order, scope) ci_sim_atomic_fetch_add((p), (v), (order))

// ---- host API -------------------------------------------------------------------------------------------------
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorLaunchFailure = 719 };
typedef struct sim_stream_ *hipStream_t;
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 1 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
struct hipDeviceProp_t {
    char gcnArchName[256];
    int multiProcessorCount;
};
static inline hipError_t hipGetDevice(int *d) {
    *d = 0;
    return hipSuccess;
}
static inline hipError_t hipDeviceGetAttribute(int *v, hipDeviceAttribute_t, int) {
    *v = sim::cu_count();
    return hipSuccess;
}
static inline hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int) {
    memset(p, 0, sizeof *p);
    strcpy(p->gcnArchName, "gfx950:host-model");
    p->multiProcessorCount = sim::cu_count();
    return hipSuccess;
}
static inline hipError_t hipFuncSetAttribute(const void *fn, hipFuncAttribute attr, int value) {
    if (attr == hipFuncAttributeMaxDynamicSharedMemorySize) sim::allow_dynamic_lds(fn, value);
    return hipSuccess;
}
static inline hipError_t hipGetLastError() { return sim::take_launch_error(); }
static inline const char *hipGetErrorString(hipError_t e) { return e ? "host model: kernel launch failed" : "no error"; }
static inline hipError_t hipMemsetAsync(void *p, int v, size_t n, hipStream_t) {
    memset(p, v, n);
    return hipSuccess;
}
static inline hipError_t hipMemcpyAsync(void *d, const void *s, size_t n, hipMemcpyKind, hipStream_t) {
    memmove(d, s, n);
    return hipSuccess;
}
static inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
#define HIP_SYMBOL(x) (sim::register_symbol((void *)&(x), sizeof(x)))
static inline hipError_t hipGetSymbolAddress(void **out, void *sym) {
    *out = sym;
    return hipSuccess;
}

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    sim::launch(#kernel, reinterpret_cast<const void *>(kernel), (grid), (block), (size_t)(shmem), [=]() { kernel(__VA_ARGS__); })
