// Small kernels that exist only in the host-model build: each makes one mistake on purpose (or none), so that the
// tests can check that the model reports it -- an address outside every allocation, an LDS address past the launch's
// LDS, a register used before the s_waitcnt that covers its load, a scalar operand that differs between lanes, lanes
// of one wavefront at different wavefront-wide operations, a workgroup that cannot go on -- and a few that pin what
// the model computes for the lane exchanges and the matrix instruction against values worked out by hand.
// Never compiled for the GPU.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

// which: 0 correct; 1 the load's offset runs 4 bytes past the array; 2 the value is used without s_waitcnt;
// 3 the base address sits in a scalar register but differs between lanes
__global__ void st_global_load_kernel(const uint32_t *src, uint32_t n, uint32_t *dst, int which) {
    const uint32_t lane = threadIdx.x;
    uint32_t off = (lane % n) * 4u + (which == 1 && lane == 7 ? n * 4u : 0u), v = 0;
    const uint64_t base = reinterpret_cast<uint64_t>(src) + (which == 3 ? (uint64_t)(lane & 1) * 4u : 0u);
    if (which == 2)
        asm volatile("global_load_dword %[v], %[off], %[base]\n"
                     "v_add_u32 %[v], %[v], %[v]\n"
                     "s_waitcnt vmcnt(0)\n"
                     : [v] "=&v"(v)
                     : [off] "v"(off), [base] "s"(base)
                     : "memory");
    else
        asm volatile("global_load_dword %[v], %[off], %[base]\n"
                     "s_waitcnt vmcnt(0)\n"
                     "v_add_u32 %[v], %[v], %[v]\n"
                     : [v] "=&v"(v)
                     : [off] "v"(off), [base] "s"(base)
                     : "memory");
    dst[lane] = v;
}

// the last byte of a large dynamic LDS area, written and read back
__global__ void st_big_lds_kernel(uint32_t *dst, uint32_t lds_bytes) {
    extern __shared__ __align__(16) uint8_t lds[];
    if (threadIdx.x == 0) lds[lds_bytes - 1] = 0x5A;
    __syncthreads();
    dst[threadIdx.x] = lds[lds_bytes - 1];
}

// which: 0 correct; 1 lane 5 reads one byte past the launch's LDS; 2 the statement ends with the read in flight
__global__ void st_lds_read_kernel(uint32_t *dst, uint32_t lds_bytes, int which) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t lane = threadIdx.x;
    lds[lane] = (uint8_t)(lane * 3u);
    __syncthreads();
    uint32_t addr = (uint32_t)(uintptr_t)lds + lane, v = 0;
    if (which == 1 && lane == 5) addr = lds_bytes;
    if (which == 2)
        asm volatile("ds_read_u8 %[v], %[a]\n" : [v] "=&v"(v) : [a] "v"(addr) : "memory");
    else
        asm volatile("ds_read_u8 %[v], %[a]\n"
                     "s_waitcnt lgkmcnt(0)\n"
                     : [v] "=&v"(v)
                     : [a] "v"(addr)
                     : "memory");
    dst[lane] = v;
}

// A masked step like the decoder's: lanes whose value is below `limit` add `add` under an execution mask.
// restore = 0 leaves the mask narrowed at the end of the statement.
__global__ void st_exec_mask_kernel(uint32_t *data, uint32_t limit, uint32_t add, int restore) {
    uint32_t v = data[threadIdx.x];
    if (restore)
        asm volatile("v_cmp_gt_u32 vcc, %[lim], %[v]\n"
                     "s_and_saveexec_b64 s[20:21], vcc\n"
                     "v_add_u32 %[v], %[add], %[v]\n"
                     "s_mov_b64 exec, s[20:21]\n"
                     : [v] "+v"(v)
                     : [lim] "s"(limit), [add] "s"(add)
                     : "vcc", "scc", "s20", "s21");
    else
        asm volatile("v_cmp_gt_u32 vcc, %[lim], %[v]\n"
                     "s_and_saveexec_b64 s[20:21], vcc\n"
                     "v_add_u32 %[v], %[add], %[v]\n"
                     : [v] "+v"(v)
                     : [lim] "s"(limit), [add] "s"(add)
                     : "vcc", "scc", "s20", "s21");
    data[threadIdx.x] = v;
}

// Lane exchanges: out[k][lane] for k = the exchanges below, of the value in[lane].
__global__ void st_lane_exchange_kernel(const uint32_t *in, uint32_t *out) {
    const uint32_t lane = threadIdx.x, x = in[lane];
    uint32_t *o = out + lane;
    o[0 * 64] = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    o[1 * 64] = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
    o[2 * 64] = (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)x, 0x104, 0xF, 0xF, false);      // row_shl:4 (old = -1)
    o[3 * 64] = (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)x, 0x114, 0xF, 0xF, false);      // row_shr:4
    o[4 * 64] = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x128, 0xF, 0xF, false);  // row_ror:8
    o[5 * 64] = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x140, 0xF, 0xF, false);  // row_mirror
    o[6 * 64] = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x141, 0xF, 0xF, false);  // row_half_mirror
    const auto s16 = __builtin_amdgcn_permlane16_swap(x, x + 1000u, false, false);
    o[7 * 64] = s16[0];
    o[8 * 64] = s16[1];
    const auto s32 = __builtin_amdgcn_permlane32_swap(x, x + 1000u, false, false);
    o[9 * 64] = s32[0];
    o[10 * 64] = s32[1];
    o[11 * 64] = (uint32_t)__builtin_amdgcn_readlane((int)x, 37);
    o[12 * 64] = (uint32_t)__builtin_amdgcn_readfirstlane((int)x);
    const uint64_t b = __builtin_amdgcn_ballot_w64((x & 1u) != 0);
    o[13 * 64] = (uint32_t)b;
    o[14 * 64] = (uint32_t)(b >> 32);
    o[15 * 64] = (uint32_t)__shfl((int)x, (int)(lane ^ 5u), 64);
    o[16 * 64] = (uint32_t)__shfl_up((int)x, 3, 64);
}

typedef __bf16 st_bf16x8 __attribute__((ext_vector_type(8)));
typedef float st_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t st_u32x4 __attribute__((ext_vector_type(4)));

// D = A B + C through the builtin (asm_form = 0) or through an assembly statement: a[i][k] and b[k][j] are plain
// bf16 matrices (32 x 16 and 16 x 32), d and c plain 32 x 32 floats; the kernel does the operand layout.
__global__ void st_mfma_kernel(const uint16_t *a, const uint16_t *b, const float *c, float *d, int asm_form) {
    const uint32_t lane = threadIdx.x, i = lane % 32, k0 = 8 * (lane / 32);
    st_u32x4 av, bv;
    for (int t = 0; t < 4; ++t) {
        av[t] = (uint32_t)a[i * 16 + k0 + 2 * t] | ((uint32_t)a[i * 16 + k0 + 2 * t + 1] << 16);
        bv[t] = (uint32_t)b[(k0 + 2 * t) * 32 + i] | ((uint32_t)b[(k0 + 2 * t + 1) * 32 + i] << 16);
    }
    st_f32x16 acc;
    for (int v = 0; v < 16; ++v) acc[v] = c[(8 * (v / 4) + 4 * (lane / 32) + v % 4) * 32 + lane % 32];
    if (asm_form)
        asm volatile("v_mfma_f32_32x32x16_bf16 %[acc], %[a], %[b], %[acc]\n"
                     "s_nop 15\n"
                     : [acc] "+v"(acc)
                     : [a] "v"(av), [b] "v"(bv));
    else
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(st_bf16x8, av), __builtin_bit_cast(st_bf16x8, bv), acc, 0, 0, 0);
    for (int v = 0; v < 16; ++v) d[(8 * (v / 4) + 4 * (lane / 32) + v % 4) * 32 + lane % 32] = acc[v];
}

// which: 0 every lane takes the ballot; 1 odd lanes take a ballot, even lanes a readfirstlane (diverged control flow
// around wavefront-wide operations: undefined on the GPU); 2 wavefront 1 skips the workgroup barrier and spins on a
// word nobody writes
__global__ void st_meeting_kernel(uint32_t *out, volatile uint32_t *never, int which) {
    const uint32_t tid = threadIdx.x;
    uint32_t r = 0;
    if (which == 1) {
        if (tid & 1)
            r = (uint32_t)__builtin_amdgcn_ballot_w64(true);
        else
            r = (uint32_t)__builtin_amdgcn_readfirstlane((int)tid);
    } else if (which == 2) {
        if (tid >= 64)
            while (*never == 0) __builtin_amdgcn_s_sleep(1);
        __syncthreads();
    } else {
        r = (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(tid % 3 == 0));
        __syncthreads();
    }
    out[tid] = r;
}

// An LDS hand-over between wavefronts through a flag and s_sleep, as the fused linear's small-M sums do it.
__global__ void st_handover_kernel(uint32_t *out) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t *word = reinterpret_cast<uint32_t *>(lds), *flag = word + 1;
    const uint32_t tid = threadIdx.x;
    if (tid == 0) *flag = 0;
    __syncthreads();
    if (tid == 64) {  // the second wavefront's first lane produces ...
        *word = 4711;
        __hip_atomic_store(flag, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (tid < 64) {  // ... the first wavefront waits for it
        while (__hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) __builtin_amdgcn_s_sleep(2);
        out[tid] = *word;
    }
}

// A plain C++ load past the end of an array: the page behind the array is inaccessible.
__global__ void st_plain_overrun_kernel(const uint32_t *src, uint32_t n, uint32_t *dst) { dst[threadIdx.x] = src[n + 16 + threadIdx.x]; }

// For the build that checks the ordering between wavefronts.  Four wavefronts each write a row of an LDS array and
// read their neighbour's; a word goes from one wavefront to another through a flag; two workgroups write the output.
// which: 0 correct; 1 no barrier between the writes and the neighbour's reads; 2 a second round of writes follows the
// reads without a barrier (write after read); 3 the flag is written and read without release / acquire; 4 the asm
// interpreter reads the neighbour's row with no barrier; 5 a `__shared__` array instead of the dynamic LDS, no barrier;
// 6 every workgroup writes the same output words; 7 workgroup 1 reads what workgroup 0 writes
__global__ void st_ordering_kernel(uint32_t *out, int which) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ uint32_t fixed[256];
    uint32_t *rows = which == 5 ? fixed : reinterpret_cast<uint32_t *>(lds), *flag = reinterpret_cast<uint32_t *>(lds) + 300,
             *word = reinterpret_cast<uint32_t *>(lds) + 1000;
    const uint32_t tid = threadIdx.x, wave = tid / 64, lane = tid % 64, next = ((wave + 1) % 4) * 64 + lane;
    rows[tid] = tid * 7u;
    if (tid == 0) *flag = 0;
    if (which != 1 && which != 4 && which != 5) __syncthreads();
    uint32_t v;
    if (which == 4) {
        __syncthreads();                       // (this one orders the first writes ...)
        rows[tid] = tid * 7u;                  // ... and these come after it, unordered with the neighbour's read below
        uint32_t b = 0;
        const uint32_t addr = (uint32_t)(uintptr_t)lds + next * 4u;
        asm volatile("ds_read_u8 %[b], %[a]\n"
                     "s_waitcnt lgkmcnt(0)\n"
                     : [b] "=&v"(b)
                     : [a] "v"(addr)
                     : "memory");
        v = b;
    } else {
        v = rows[next];
    }
    if (which == 2) rows[tid] = v;  // the neighbour may not have read this row yet
    if (which == 0) {
        __syncthreads();
        rows[tid] = v;
    }
    __syncthreads();
    // a word handed from wavefront 1 to wavefront 0
    if (tid == 64) {
        *word = 4711;
        if (which == 3)
            __hip_atomic_store(flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else
            __hip_atomic_store(flag, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (tid < 64) {
        if (which == 3)
            while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) __builtin_amdgcn_s_sleep(2);
        else
            while (__hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == 0) __builtin_amdgcn_s_sleep(2);
        v += *word;
    }
    if (which == 7 && blockIdx.x == 1) v += out[tid];
    out[(which == 6 || which == 7 ? 0u : blockIdx.x) * blockDim.x + tid] = v;
}

// A running sum handed from lane to lane through the LDS: right when the lanes run one after the other, as they do in
// the model, and wrong on the GPU, where they run in step.  which: 0 every lane writes its own word, a wavefront-wide
// operation, then reads its neighbour's (well defined); 1 lane l adds what lane l - 1 has just stored, with nothing
// wavefront-wide between the store and the load; 2 the same through the output array instead of the LDS
__global__ void st_lane_order_kernel(uint32_t *out, int which) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t *word = reinterpret_cast<uint32_t *>(lds);
    const uint32_t lane = threadIdx.x;
    if (which == 0) {
        word[lane] = lane + 1;
        __builtin_amdgcn_wave_barrier();
        out[lane] = word[lane] + (lane ? word[lane - 1] : 0u);
    } else if (which == 1) {
        const uint32_t before = lane ? word[lane - 1] : 0u;
        word[lane] = before + lane + 1;
        out[lane] = word[lane];
    } else {
        out[lane] = (lane ? out[lane - 1] : 0u) + lane + 1;
    }
}

// For the build with the compiler's undefined-behaviour checks.  which: 0 nothing; 1 a shift by the width of the
// type; 2 an index one past a fixed-size array; 3 a 16-byte access at an address that is a multiple of 4 only;
// 4 a signed sum past the largest int
typedef uint32_t st_u32x4 __attribute__((ext_vector_type(4)));
__global__ void st_undefined_kernel(uint32_t *out, int which, uint32_t n) {  // n = 32
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t tid = threadIdx.x;
    uint32_t regs[4] = {tid, tid + 1, tid + 2, tid + 3};
    uint32_t v = regs[(tid + n) % 4];
    if (which == 1) v += 1u << n;
    static const uint32_t table[4] = {3, 1, 4, 1};  // (in memory: the access past it goes on after the report)
    if (which == 2) v += table[n / 8];
    for (uint32_t i = 0; i < 8; ++i) reinterpret_cast<uint32_t *>(lds)[tid * 8 + i] = i;
    if (which == 3) v += (*reinterpret_cast<const st_u32x4 *>(lds + tid * 32 + n / 8))[1];
    if (which == 4) v += (uint32_t)((int)(0x7fffffe0u + tid) + (int)n);
    out[tid] = v;
}

}  // namespace

extern "C" {
void simtest_lane_order(uint32_t *out, int which) { hipLaunchKernelGGL(st_lane_order_kernel, dim3(1), dim3(64), 256, nullptr, out, which); }
void simtest_undefined(uint32_t *out, int which, uint32_t n) {
    hipLaunchKernelGGL(st_undefined_kernel, dim3(1), dim3(64), 4096, nullptr, out, which, n);
}
void simtest_ordering(uint32_t *out, int which) {
    hipLaunchKernelGGL(st_ordering_kernel, dim3(2), dim3(256), 8192, nullptr, out, which);
}
void simtest_global_load(const uint32_t *src, uint32_t n, uint32_t *dst, int which) {
    hipLaunchKernelGGL(st_global_load_kernel, dim3(1), dim3(64), 0, nullptr, src, n, dst, which);
}
// allowed: whether hipFuncSetAttribute is called first, as a launch with more than 64 KB of dynamic LDS needs
void simtest_big_lds(uint32_t *dst, uint32_t lds_bytes, int allowed) {
    if (allowed) (void)hipFuncSetAttribute(reinterpret_cast<const void *>(st_big_lds_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    hipLaunchKernelGGL(st_big_lds_kernel, dim3(1), dim3(64), lds_bytes, nullptr, dst, lds_bytes);
}
void simtest_lds_read(uint32_t *dst, uint32_t lds_bytes, int which) {
    hipLaunchKernelGGL(st_lds_read_kernel, dim3(1), dim3(64), lds_bytes, nullptr, dst, lds_bytes, which);
}
void simtest_exec_mask(uint32_t *data, uint32_t limit, uint32_t add, int restore) {
    hipLaunchKernelGGL(st_exec_mask_kernel, dim3(1), dim3(64), 0, nullptr, data, limit, add, restore);
}
void simtest_lane_exchange(const uint32_t *in, uint32_t *out) {
    hipLaunchKernelGGL(st_lane_exchange_kernel, dim3(1), dim3(64), 0, nullptr, in, out);
}
void simtest_mfma(const uint16_t *a, const uint16_t *b, const float *c, float *d, int asm_form) {
    hipLaunchKernelGGL(st_mfma_kernel, dim3(1), dim3(64), 0, nullptr, a, b, c, d, asm_form);
}
void simtest_meeting(uint32_t *out, uint32_t *never, int which) {
    hipLaunchKernelGGL(st_meeting_kernel, dim3(1), dim3(128), 0, nullptr, out, never, which);
}
void simtest_handover(uint32_t *out) { hipLaunchKernelGGL(st_handover_kernel, dim3(1), dim3(128), 64, nullptr, out); }
void simtest_plain_overrun(const uint32_t *src, uint32_t n, uint32_t *dst) {
    hipLaunchKernelGGL(st_plain_overrun_kernel, dim3(1), dim3(64), 0, nullptr, src, n, dst);
}
}
