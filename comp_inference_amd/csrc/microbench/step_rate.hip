// Step-rate microbenchmark: what one rANS decode step of one wavefront (64 streams) costs a CU, for several
// formulations of the step and from 1 to 16 wavefronts per CU.  Stand-alone program (HIP runtime only):
//
//     python -m comp_inference_amd.build --microbench      -> comp_inference_amd/step_rate_bench
//     ./comp_inference_amd/step_rate_bench
//
// Streams are real: exponents of bf16 N(0, 0.02) values, 12-bit tables, 128 steps per stream, encoded on the
// host; every variant decodes whole streams out of LDS-staged bodies and is checked against a host decoder
// (a table checksum per lane and the final state 2^16).  The kernels of the library take their step from
// here: `masked` is the step of csrc/fast_tile.h.  Columns of the second table:
//   old-3-LDS         two bytes read ahead every step, both renormalisations by v_cndmask (three LDS reads)
//   masked            one byte under an execution mask, the rare second byte out of line (the shipped step)
//   x256 ...          the same ideas with the state scaled by 256 instead of 8 (address by v_bfe, byte by v_perm)
//   masked 2 chains   two independent streams per lane, interleaved
//   branch-free       one byte by v_cndmask, the rare second byte looked for one step later
// The first table is the raw cost of the LDS reads a step is made of.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <vector>
#include <random>
#define CK(x) do{hipError_t err_=(x); if(err_!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(err_), __LINE__); exit(1);} }while(0)

constexpr int kHalf = 128;          // steps per stream
constexpr int kStr = 60;            // LDS bytes per lane (15 dwords)
constexpr int kTiles = 64;
constexpr uint32_t kL = 1u << 16;

struct Args {
    const uint2 *tab64; const uint32_t *tab32; const uint2 *tab256;
    const uint8_t *bodies;      // [kTiles][kStr][64] rows of 64 bytes, row r at r*64
    const uint32_t *depth;      // [kTiles]
    const uint32_t *states;     // [kTiles][64]
    uint32_t *out;              // [blocks*threads][2]
    int passes;
};

// V: 0 shipping step, 1 exec-masked single-byte step with rare second byte (8-byte table),
//    2 the same with a 4-byte table, 3 = 1 without the rare check (wrong results, cost of the check),
//    4 = 1 with the byte read issued for every lane (not masked)
template <int V>
__global__ __launch_bounds__(1024) void step_kernel(Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    constexpr uint32_t kTabBytes = (V == 2) ? 16384 : 32768;
    if (V == 2) { for (int s = tid; s < 4096; s += blockDim.x) ((uint32_t *)lds)[s] = a.tab32[s]; }
    else if (V >= 5) { for (int s = tid; s < 4096; s += blockDim.x) ((uint2 *)lds)[s] = a.tab256[s]; }
    else { for (int s = tid; s < 4096; s += blockDim.x) ((uint2 *)lds)[s] = a.tab64[s]; }
    const int tile = (blockIdx.x * 16 + wave) % kTiles;
    uint8_t *stage = lds + kTabBytes + wave * 64 * kStr;
    const uint32_t depth = a.depth[tile];
    for (uint32_t r = 0; r < depth; ++r) stage[lane * kStr + r] = a.bodies[((size_t)tile * kStr + r) * 64 + lane];
    __syncthreads();
    const uint32_t state0 = a.states[tile * 64 + lane];
    const uint32_t col = (uint32_t)(uintptr_t)(stage + lane * kStr);
    uint32_t acc = 0, Xfin = 0;
    for (int p = 0; p < a.passes; ++p) {
        if (V == 0) {
            uint32_t X = state0 << 3, q = col + depth - 2, n1 = stage[lane * kStr + depth - 1], n2 = depth >= 2 ? stage[lane * kStr + depth - 2] : 0;
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                "v_and_b32 v76, 0x7ff8, %[X]\n"
                "ds_read_b64 v[72:73], v76\n"
                "v_lshrrev_b32 v77, 15, %[X]\n"
                "s_waitcnt lgkmcnt(1)\n"
                "v_lshlrev_b32 v78, 3, %[n1]\n"
                "v_lshlrev_b32 v79, 3, %[n2]\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_mad_u32_u24 v80, v72, v77, v73\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L8], v80\n"
                "v_cmp_gt_u32 s[20:21], %[B8], v80\n"
                "v_lshl_or_b32 v81, v80, 8, v78\n"
                "v_lshl_or_b32 v82, v81, 8, v79\n"
                "v_cndmask_b32 %[X], v80, v81, vcc\n"
                "v_subbrev_co_u32 %[q], vcc, 0, %[q], vcc\n"
                "v_cndmask_b32 %[X], %[X], v82, s[20:21]\n"
                "v_subbrev_co_u32 %[q], vcc, 0, %[q], s[20:21]\n"
                "ds_read_u8 %[n1], %[q] offset:1\n"
                "ds_read_u8 %[n2], %[q]\n"
                "s_sub_u32 s22, s22, 1\n"
                "s_cmp_lg_u32 s22, 0\n"
                "s_cbranch_scc1 1b\n"
                "s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [n2] "+v"(n2), [acc] "+v"(acc)
                : [L8] "s"(kL << 3), [B8] "s"(256u << 3)
                : "vcc", "scc", "s20", "s21", "s22", "v72", "v73", "v76", "v77", "v78", "v79", "v80", "v81", "v82", "memory");
            Xfin = X >> 3;
        } else if (V == 1 || V == 3 || V == 4) {
            uint32_t X = state0 << 3, q = col + depth - 1, n1 = stage[lane * kStr + depth - 1];
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                "v_and_b32 v76, 0x7ff8, %[X]\n"
                "ds_read_b64 v[72:73], v76\n"
                "v_lshrrev_b32 v77, 15, %[X]\n"
                "s_waitcnt lgkmcnt(1)\n"
                "v_lshlrev_b32 v78, 3, %[n1]\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_mad_u32_u24 %[X], v72, v77, v73\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L8], %[X]\n"
                "s_and_saveexec_b64 s[20:21], vcc\n"
                "v_lshl_or_b32 %[X], %[X], 8, v78\n"
                "v_add_u32 %[q], -1, %[q]\n"
                ".if %c[V] != 4\n ds_read_u8 %[n1], %[q]\n .endif\n"
                ".if %c[V] != 3\n"
                "v_cmpx_gt_u32 vcc, %[L8], %[X]\n"
                "s_cbranch_execnz 3f\n"
                ".endif\n"
                "2:\n"
                "s_mov_b64 exec, s[20:21]\n"
                ".if %c[V] == 4\n ds_read_u8 %[n1], %[q]\n .endif\n"
                "s_sub_u32 s22, s22, 1\n"
                "s_cmp_lg_u32 s22, 0\n"
                "s_cbranch_scc1 1b\n"
                "s_branch 4f\n"
                "3:\n"
                ".if %c[V] == 4\n ds_read_u8 %[n1], %[q]\n .endif\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_lshlrev_b32 v78, 3, %[n1]\n"
                "v_lshl_or_b32 %[X], %[X], 8, v78\n"
                "v_add_u32 %[q], -1, %[q]\n"
                ".if %c[V] != 4\n ds_read_u8 %[n1], %[q]\n .endif\n"
                "s_branch 2b\n"
                "4:\n"
                "s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [acc] "+v"(acc)
                : [L8] "s"(kL << 3), [V] "n"(V)
                : "vcc", "scc", "s20", "s21", "s22", "v72", "v73", "v76", "v77", "v78", "memory");
            Xfin = X >> 3;
        } else if (V == 2) {
            // unscaled state, 4-byte entries sym<<24 | freq<<12 | (slot - cdf)
            uint32_t X = state0, q = col + depth - 1, n1 = stage[lane * kStr + depth - 1];
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                "v_and_b32 v76, 0xfff, %[X]\n"
                "v_lshlrev_b32 v76, 2, v76\n"
                "ds_read_b32 v72, v76\n"
                "v_lshrrev_b32 v77, 12, %[X]\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_bfe_u32 v73, v72, 12, 12\n"
                "v_and_b32 v74, 0xfff, v72\n"
                "v_mad_u32_u24 %[X], v73, v77, v74\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L], %[X]\n"
                "s_and_saveexec_b64 s[20:21], vcc\n"
                "v_lshl_or_b32 %[X], %[X], 8, %[n1]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "v_cmpx_gt_u32 vcc, %[L], %[X]\n"
                "s_cbranch_execnz 3f\n"
                "2:\n"
                "s_mov_b64 exec, s[20:21]\n"
                "s_sub_u32 s22, s22, 1\n"
                "s_cmp_lg_u32 s22, 0\n"
                "s_cbranch_scc1 1b\n"
                "s_branch 4f\n"
                "3:\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_lshl_or_b32 %[X], %[X], 8, %[n1]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "s_branch 2b\n"
                "4:\n"
                "s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [acc] "+v"(acc)
                : [L] "s"(kL)
                : "vcc", "scc", "s20", "s21", "s22", "v72", "v73", "v74", "v76", "v77", "memory");
            Xfin = X;
        } else if (V == 5) {
            // state scaled by 256: address by one bit-field extract, byte inserted by one byte permute; branch-free
            uint32_t X = state0 << 8, q = col + depth - 1, n1 = stage[lane * kStr + depth - 1];
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                "v_bfe_u32 v76, %[X], 5, 15\n"
                "ds_read_b64 v[72:73], v76\n"
                "v_lshrrev_b32 v77, 20, %[X]\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_mad_u32_u24 v80, v72, v77, v73\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L], v80\n"
                "v_perm_b32 v81, v80, %[n1], %[sel]\n"
                "v_cndmask_b32 %[X], v80, v81, vcc\n"
                "v_subbrev_co_u32 %[q], vcc, 0, %[q], vcc\n"
                "ds_read_u8 %[n1], %[q]\n"
                "v_cmp_gt_u32 vcc, %[L], %[X]\n"
                "s_cbranch_vccnz 3f\n"
                "2:\n"
                "s_sub_u32 s22, s22, 1\n"
                "s_cmp_lg_u32 s22, 0\n"
                "s_cbranch_scc1 1b\n"
                "s_branch 4f\n"
                "3:\n"
                "s_and_saveexec_b64 s[20:21], vcc\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_perm_b32 %[X], %[X], %[n1], %[sel]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "s_mov_b64 exec, s[20:21]\n"
                "s_branch 2b\n"
                "4:\n"
                "s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [acc] "+v"(acc)
                : [L] "s"(kL << 8), [sel] "s"(0x0605000Cu)
                : "vcc", "scc", "s20", "s21", "s22", "v72", "v73", "v76", "v77", "v80", "v81", "memory");
            Xfin = X >> 8;
        } else if (V == 6) {
            // the same under an execution mask
            uint32_t X = state0 << 8, q = col + depth - 1, n1 = stage[lane * kStr + depth - 1];
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                "v_bfe_u32 v76, %[X], 5, 15\n"
                "ds_read_b64 v[72:73], v76\n"
                "v_lshrrev_b32 v77, 20, %[X]\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_mad_u32_u24 %[X], v72, v77, v73\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L], %[X]\n"
                "s_and_saveexec_b64 s[20:21], vcc\n"
                "v_perm_b32 %[X], %[X], %[n1], %[sel]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "v_cmpx_gt_u32 vcc, %[L], %[X]\n"
                "s_cbranch_execnz 3f\n"
                "2:\n"
                "s_mov_b64 exec, s[20:21]\n"
                "s_sub_u32 s22, s22, 1\n"
                "s_cmp_lg_u32 s22, 0\n"
                "s_cbranch_scc1 1b\n"
                "s_branch 4f\n"
                "3:\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_perm_b32 %[X], %[X], %[n1], %[sel]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "s_branch 2b\n"
                "4:\n"
                "s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [acc] "+v"(acc)
                : [L] "s"(kL << 8), [sel] "s"(0x0605000Cu)
                : "vcc", "scc", "s20", "s21", "s22", "v72", "v73", "v76", "v77", "memory");
            Xfin = X >> 8;
        } else if (V == 7) {
            // x256 state, branch-free, the rare second byte looked for one step later (after the next table read
            // has been issued; a lane that needed it gets its byte and the read is issued again)
            uint32_t X = state0 << 8, q = col + depth - 1, n1 = stage[lane * kStr + depth - 1];
            asm volatile(
                "s_movk_i32 s22, 128\n s_mov_b64 s[24:25], 0\n"
                "1:\n"
                "v_bfe_u32 v76, %[X], 5, 15\n"
                "ds_read_b64 v[72:73], v76\n"
                "v_lshrrev_b32 v77, 20, %[X]\n"
                "s_cmp_lg_u64 s[24:25], 0\n s_cbranch_scc1 8f\n"
                "s_waitcnt lgkmcnt(0)\n"
                "v_mad_u32_u24 v80, v72, v77, v73\n"
                "v_add_u32 %[acc], %[acc], v72\n"
                "v_cmp_gt_u32 vcc, %[L], v80\n"
                "v_perm_b32 v81, v80, %[n1], %[sel]\n"
                "v_cndmask_b32 %[X], v80, v81, vcc\n"
                "v_subbrev_co_u32 %[q], vcc, 0, %[q], vcc\n"
                "ds_read_u8 %[n1], %[q]\n"
                "v_cmp_gt_u32 s[24:25], %[L], %[X]\n"
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "s_cmp_lg_u64 s[24:25], 0\n s_cbranch_scc0 7f\n s_movk_i32 s22, 0\n"
                "8:\n"
                "s_mov_b64 s[20:21], exec\n s_waitcnt lgkmcnt(0)\n"
                "s_mov_b64 exec, s[24:25]\n"
                "v_perm_b32 %[X], %[X], %[n1], %[sel]\n"
                "v_add_u32 %[q], -1, %[q]\n"
                "ds_read_u8 %[n1], %[q]\n"
                "s_mov_b64 exec, s[20:21]\n s_mov_b64 s[24:25], 0\n"
                "s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "7:\n s_waitcnt lgkmcnt(0)\n"
                : [X] "+v"(X), [q] "+v"(q), [n1] "+v"(n1), [acc] "+v"(acc)
                : [L] "s"(kL << 8), [sel] "s"(0x0605000Cu)
                : "vcc", "scc", "s20", "s21", "s22", "s24", "s25", "v72", "v73", "v76", "v77", "v80", "v81", "memory");
            Xfin = X >> 8;
        }
    }
    a.out[(blockIdx.x * blockDim.x + tid) * 2] = acc;
    a.out[(blockIdx.x * blockDim.x + tid) * 2 + 1] = Xfin;
}

// Raw LDS throughput: K 0 random 8-byte reads, 1 random 4-byte reads, 2 byte reads at per-lane columns,
// 3 8-byte reads all lanes one address.
template <int K>
__global__ __launch_bounds__(1024) void lds_kernel(uint32_t *out, int iters) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid % 64;
    for (int s = tid; s < 8192; s += blockDim.x) ((uint32_t *)lds)[s] = s * 2654435761u;
    __syncthreads();
    uint32_t addr = (tid * 2654435761u >> 7), acc = 0;
    if (K == 2) addr = lane * 116 + (tid * 7 % 13);
    for (int i = 0; i < iters; ++i) {
        asm volatile(
            ".rept 8\n"
            ".if %c[K] == 0\n v_mad_u32_u24 %[a], %[a], 5, 56\n v_and_b32 v76, 0x7ff8, %[a]\n ds_read_b64 v[72:73], v76\n .endif\n"
            ".if %c[K] == 1\n v_mad_u32_u24 %[a], %[a], 5, 60\n v_and_b32 v76, 0x3ffc, %[a]\n ds_read_b32 v72, v76\n .endif\n"
            ".if %c[K] == 2\n v_add_u32 %[a], 1, %[a]\n v_and_b32 v76, 0x1fff, %[a]\n ds_read_u8 v72, v76\n .endif\n"
            ".if %c[K] == 3\n v_mad_u32_u24 %[a], %[a], 5, 56\n v_and_b32 v76, 0x0, %[a]\n ds_read_b64 v[72:73], v76\n .endif\n"
            ".endr\n"
            "s_waitcnt lgkmcnt(0)\n"
            "v_add_u32 %[acc], %[acc], v72\n"
            : [a] "+v"(addr), [acc] "+v"(acc) : [K] "n"(K) : "v72", "v73", "v76", "memory");
    }
    out[blockIdx.x * blockDim.x + tid] = acc;
}


// C independent chains per wavefront, written in C++ and scheduled by the compiler.
template <int C>
__global__ __launch_bounds__(1024) void cpp_kernel(Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    for (int s = tid; s < 4096; s += blockDim.x) ((uint2 *)lds)[s] = a.tab64[s];
    uint32_t depth[C], state0[C], col[C];
    int tile[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        tile[c] = ((blockIdx.x * 16 + wave) * C + c) % kTiles;
        uint8_t *stage = lds + 32768 + (wave * C + c) * 64 * kStr;
        depth[c] = a.depth[tile[c]];
        for (uint32_t r = 0; r < depth[c]; ++r) stage[lane * kStr + r] = a.bodies[((size_t)tile[c] * kStr + r) * 64 + lane];
        state0[c] = a.states[tile[c] * 64 + lane];
        col[c] = (uint32_t)(uintptr_t)(stage + lane * kStr);
    }
    __syncthreads();
    uint32_t acc[C], Xf[C];
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = 0;
    for (int p = 0; p < a.passes; ++p) {
        uint32_t X[C], q[C], n1[C];
#pragma unroll
        for (int c = 0; c < C; ++c) { X[c] = state0[c] << 3; q[c] = col[c] + depth[c] - 1; n1[c] = lds[q[c]]; }
        for (int i = 0; i < kHalf; i += 4) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    const uint2 e = *reinterpret_cast<const uint2 *>(lds + (X[c] & 0x7ff8u));
                    acc[c] += e.x;
                    X[c] = __umul24(e.x, X[c] >> 15) + e.y;
                    if (X[c] < (kL << 3)) { X[c] = (X[c] << 8) | (n1[c] << 3); q[c] -= 1; n1[c] = lds[q[c]]; }
                }
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    if (__builtin_amdgcn_ballot_w64(X[c] < (kL << 3)) != 0) {
                        if (X[c] < (kL << 3)) { X[c] = (X[c] << 8) | (n1[c] << 3); q[c] -= 1; n1[c] = lds[q[c]]; }
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c) Xf[c] = X[c] >> 3;
    }
#pragma unroll
    for (int c = 0; c < C; ++c) {
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2] = acc[c];
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2 + 1] = Xf[c];
    }
}


#define MC_ISSUE(c, E)  "v_and_b32 v6" #c ", 0x7ff8, %[X" #c "]\n ds_read_b64 " E ", v6" #c "\n v_lshrrev_b32 v7" #c ", 15, %[X" #c "]\n"
#define MC_SHIFT(c)     "v_lshlrev_b32 v8" #c ", 3, %[n" #c "]\n"
#define MC_FINISH(c, ELO, EHI, WAIT)                       \
    "s_waitcnt lgkmcnt(" WAIT ")\n"                        \
    "v_mad_u32_u24 %[X" #c "], " ELO ", v7" #c ", " EHI "\n" \
    "v_add_u32 %[acc" #c "], %[acc" #c "], " ELO "\n"      \
    "v_cmp_gt_u32 vcc, %[L8], %[X" #c "]\n"               \
    "s_and_saveexec_b64 s[20:21], vcc\n"                   \
    "v_lshl_or_b32 %[X" #c "], %[X" #c "], 8, v8" #c "\n" \
    "v_add_u32 %[q" #c "], -1, %[q" #c "]\n"               \
    "ds_read_u8 %[n" #c "], %[q" #c "]\n"                  \
    "v_cmpx_gt_u32 vcc, %[L8], %[X" #c "]\n"               \
    "s_cbranch_execnz 8f\n"                                \
    "9:\n"                                                 \
    "s_mov_b64 exec, s[20:21]\n"                           \
    ".subsection 1\n"                                      \
    "8:\n"                                                 \
    "s_waitcnt lgkmcnt(0)\n"                               \
    "v_lshlrev_b32 v8" #c ", 3, %[n" #c "]\n"             \
    "v_lshl_or_b32 %[X" #c "], %[X" #c "], 8, v8" #c "\n" \
    "v_add_u32 %[q" #c "], -1, %[q" #c "]\n"               \
    "ds_read_u8 %[n" #c "], %[q" #c "]\n"                  \
    "s_branch 9b\n"                                        \
    ".subsection 0\n"

// C chains per wavefront, hand-interleaved: all table reads of a step in flight together.
template <int C>
__global__ __launch_bounds__(1024) void mc_kernel(Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    for (int s = tid; s < 4096; s += blockDim.x) ((uint2 *)lds)[s] = a.tab64[s];
    uint32_t depth[4], state0[4], col[4];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int tile = ((blockIdx.x * 16 + wave) * C + c) % kTiles;
        uint8_t *stage = lds + 32768 + (wave * C + c) * 64 * kStr;
        depth[c] = a.depth[tile];
        for (uint32_t r = 0; r < depth[c]; ++r) stage[lane * kStr + r] = a.bodies[((size_t)tile * kStr + r) * 64 + lane];
        state0[c] = a.states[tile * 64 + lane];
        col[c] = (uint32_t)(uintptr_t)(stage + lane * kStr);
    }
    __syncthreads();
    uint32_t acc[4] = {0, 0, 0, 0}, X[4] = {0, 0, 0, 0}, q[4] = {0, 0, 0, 0}, n1[4] = {0, 0, 0, 0};
    for (int p = 0; p < a.passes; ++p) {
#pragma unroll
        for (int c = 0; c < C; ++c) { X[c] = state0[c] << 3; q[c] = col[c] + depth[c] - 1; n1[c] = lds[q[c]]; }
        if (C == 2) {
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                MC_ISSUE(0, "v[90:91]") MC_ISSUE(1, "v[92:93]")
                "s_waitcnt lgkmcnt(2)\n" MC_SHIFT(0) MC_SHIFT(1)
                MC_FINISH(0, "v90", "v91", "1") MC_FINISH(1, "v92", "v93", "1")
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n s_waitcnt lgkmcnt(0)\n"
                : [X0] "+v"(X[0]), [q0] "+v"(q[0]), [n0] "+v"(n1[0]), [acc0] "+v"(acc[0]),
                  [X1] "+v"(X[1]), [q1] "+v"(q[1]), [n1] "+v"(n1[1]), [acc1] "+v"(acc[1])
                : [L8] "s"(kL << 3)
                : "vcc", "scc", "s20", "s21", "s22", "v60", "v61", "v70", "v71", "v80", "v81", "v90", "v91", "v92", "v93", "memory");
        } else if (C == 4) {
            asm volatile(
                "s_movk_i32 s22, 128\n"
                "1:\n"
                MC_ISSUE(0, "v[90:91]") MC_ISSUE(1, "v[92:93]") MC_ISSUE(2, "v[94:95]") MC_ISSUE(3, "v[96:97]")
                "s_waitcnt lgkmcnt(4)\n" MC_SHIFT(0) MC_SHIFT(1) MC_SHIFT(2) MC_SHIFT(3)
                MC_FINISH(0, "v90", "v91", "3") MC_FINISH(1, "v92", "v93", "3") MC_FINISH(2, "v94", "v95", "3") MC_FINISH(3, "v96", "v97", "3")
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n s_waitcnt lgkmcnt(0)\n"
                : [X0] "+v"(X[0]), [q0] "+v"(q[0]), [n0] "+v"(n1[0]), [acc0] "+v"(acc[0]),
                  [X1] "+v"(X[1]), [q1] "+v"(q[1]), [n1] "+v"(n1[1]), [acc1] "+v"(acc[1]),
                  [X2] "+v"(X[2]), [q2] "+v"(q[2]), [n2] "+v"(n1[2]), [acc2] "+v"(acc[2]),
                  [X3] "+v"(X[3]), [q3] "+v"(q[3]), [n3] "+v"(n1[3]), [acc3] "+v"(acc[3])
                : [L8] "s"(kL << 3)
                : "vcc", "scc", "s20", "s21", "s22", "v60", "v61", "v62", "v63", "v70", "v71", "v72", "v73", "v80", "v81", "v82", "v83",
                  "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "memory");
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c) {
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2] = acc[c];
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2 + 1] = X[c] >> 3;
    }
}


// Branch-free single-byte step; the rare second byte is found by a compare whose result is looked at one
// step later, after the next table reads have been issued.
#define BF_ISSUE(c, E)  "v_and_b32 v6" #c ", 0x7ff8, %[X" #c "]\n ds_read_b64 " E ", v6" #c "\n v_lshrrev_b32 v7" #c ", 15, %[X" #c "]\n"
#define BF_SHIFT(c)     "v_lshlrev_b32 v8" #c ", 3, %[n" #c "]\n"
#define BF_FINISH(c, ELO, EHI, WAIT, RS)                   \
    "s_waitcnt lgkmcnt(" WAIT ")\n"                        \
    "v_mad_u32_u24 v5" #c ", " ELO ", v7" #c ", " EHI "\n" \
    "v_add_u32 %[acc" #c "], %[acc" #c "], " ELO "\n"      \
    "v_lshl_or_b32 v4" #c ", v5" #c ", 8, v8" #c "\n"     \
    "v_cmp_gt_u32 vcc, %[L8], v5" #c "\n"                 \
    "v_cndmask_b32 %[X" #c "], v5" #c ", v4" #c ", vcc\n" \
    "v_subbrev_co_u32 %[q" #c "], vcc, 0, %[q" #c "], vcc\n" \
    "ds_read_u8 %[n" #c "], %[q" #c "]\n"                  \
    "v_cmp_gt_u32 " RS ", %[L8], %[X" #c "]\n"
#define BF_FIX(c, RS)                                      \
    "s_mov_b64 exec, " RS "\n"                             \
    "v_lshlrev_b32 v8" #c ", 3, %[n" #c "]\n"             \
    "v_lshl_or_b32 %[X" #c "], %[X" #c "], 8, v8" #c "\n" \
    "v_add_u32 %[q" #c "], -1, %[q" #c "]\n"               \
    "ds_read_u8 %[n" #c "], %[q" #c "]\n"

template <int C>
__global__ __launch_bounds__(1024) void bf_kernel(Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    for (int s = tid; s < 4096; s += blockDim.x) ((uint2 *)lds)[s] = a.tab64[s];
    uint32_t depth[4], state0[4], col[4];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int tile = ((blockIdx.x * 16 + wave) * C + c) % kTiles;
        uint8_t *stage = lds + 32768 + (wave * C + c) * 64 * kStr;
        depth[c] = a.depth[tile];
        for (uint32_t r = 0; r < depth[c]; ++r) stage[lane * kStr + r] = a.bodies[((size_t)tile * kStr + r) * 64 + lane];
        state0[c] = a.states[tile * 64 + lane];
        col[c] = (uint32_t)(uintptr_t)(stage + lane * kStr);
    }
    __syncthreads();
    uint32_t acc[4] = {0, 0, 0, 0}, X[4] = {0, 0, 0, 0}, q[4] = {0, 0, 0, 0}, n1[4] = {0, 0, 0, 0};
    for (int p = 0; p < a.passes; ++p) {
#pragma unroll
        for (int c = 0; c < C; ++c) { X[c] = state0[c] << 3; q[c] = col[c] + depth[c] - 1; n1[c] = lds[q[c]]; }
        if (C == 1) {
            asm volatile(
                "s_movk_i32 s22, 128\n s_mov_b64 s[24:25], 0\n"
                "1:\n"
                BF_ISSUE(0, "v[90:91]")
                "s_cmp_lg_u64 s[24:25], 0\n s_cbranch_scc1 8f\n"
                "s_waitcnt lgkmcnt(1)\n" BF_SHIFT(0)
                BF_FINISH(0, "v90", "v91", "0", "s[24:25]")
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "s_cmp_lg_u64 s[24:25], 0\n s_cbranch_scc0 7f\n s_movk_i32 s22, 0\n"
                "8:\n"
                "s_mov_b64 s[20:21], exec\n s_waitcnt lgkmcnt(0)\n"
                BF_FIX(0, "s[24:25]")
                "s_mov_b64 exec, s[20:21]\n s_mov_b64 s[24:25], 0\n"
                "s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "7:\n s_waitcnt lgkmcnt(0)\n"
                : [X0] "+v"(X[0]), [q0] "+v"(q[0]), [n0] "+v"(n1[0]), [acc0] "+v"(acc[0])
                : [L8] "s"(kL << 3)
                : "vcc", "scc", "s20", "s21", "s22", "s24", "s25", "v40", "v50", "v60", "v70", "v80", "v90", "v91", "memory");
        } else if (C == 2) {
            asm volatile(
                "s_movk_i32 s22, 128\n s_mov_b64 s[24:25], 0\n s_mov_b64 s[26:27], 0\n"
                "1:\n"
                BF_ISSUE(0, "v[90:91]") BF_ISSUE(1, "v[92:93]")
                "s_or_b64 s[30:31], s[24:25], s[26:27]\n s_cmp_lg_u64 s[30:31], 0\n s_cbranch_scc1 8f\n"
                "s_waitcnt lgkmcnt(2)\n" BF_SHIFT(0) BF_SHIFT(1)
                BF_FINISH(0, "v90", "v91", "1", "s[24:25]") BF_FINISH(1, "v92", "v93", "1", "s[26:27]")
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "s_or_b64 s[30:31], s[24:25], s[26:27]\n s_cmp_lg_u64 s[30:31], 0\n s_cbranch_scc0 7f\n s_movk_i32 s22, 0\n"
                "8:\n"
                "s_mov_b64 s[20:21], exec\n s_waitcnt lgkmcnt(0)\n"
                BF_FIX(0, "s[24:25]") BF_FIX(1, "s[26:27]")
                "s_mov_b64 exec, s[20:21]\n s_mov_b64 s[24:25], 0\n s_mov_b64 s[26:27], 0\n"
                "s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "7:\n s_waitcnt lgkmcnt(0)\n"
                : [X0] "+v"(X[0]), [q0] "+v"(q[0]), [n0] "+v"(n1[0]), [acc0] "+v"(acc[0]),
                  [X1] "+v"(X[1]), [q1] "+v"(q[1]), [n1] "+v"(n1[1]), [acc1] "+v"(acc[1])
                : [L8] "s"(kL << 3)
                : "vcc", "scc", "s20", "s21", "s22", "s24", "s25", "s26", "s27", "s30", "s31", "v40", "v41", "v50", "v51", "v60", "v61", "v70", "v71",
                  "v80", "v81", "v90", "v91", "v92", "v93", "memory");
        } else if (C == 4) {
            asm volatile(
                "s_movk_i32 s22, 128\n s_mov_b64 s[24:25], 0\n s_mov_b64 s[26:27], 0\n s_mov_b64 s[28:29], 0\n s_mov_b64 s[34:35], 0\n"
                "1:\n"
                BF_ISSUE(0, "v[90:91]") BF_ISSUE(1, "v[92:93]") BF_ISSUE(2, "v[94:95]") BF_ISSUE(3, "v[96:97]")
                "s_or_b64 s[30:31], s[24:25], s[26:27]\n s_or_b64 s[30:31], s[30:31], s[28:29]\n s_or_b64 s[30:31], s[30:31], s[34:35]\n"
                "s_cmp_lg_u64 s[30:31], 0\n s_cbranch_scc1 8f\n"
                "s_waitcnt lgkmcnt(4)\n" BF_SHIFT(0) BF_SHIFT(1) BF_SHIFT(2) BF_SHIFT(3)
                BF_FINISH(0, "v90", "v91", "3", "s[24:25]") BF_FINISH(1, "v92", "v93", "3", "s[26:27]")
                BF_FINISH(2, "v94", "v95", "3", "s[28:29]") BF_FINISH(3, "v96", "v97", "3", "s[34:35]")
                "s_sub_u32 s22, s22, 1\n s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "s_or_b64 s[30:31], s[24:25], s[26:27]\n s_or_b64 s[30:31], s[30:31], s[28:29]\n s_or_b64 s[30:31], s[30:31], s[34:35]\n"
                "s_cmp_lg_u64 s[30:31], 0\n s_cbranch_scc0 7f\n s_movk_i32 s22, 0\n"
                "8:\n"
                "s_mov_b64 s[20:21], exec\n s_waitcnt lgkmcnt(0)\n"
                BF_FIX(0, "s[24:25]") BF_FIX(1, "s[26:27]") BF_FIX(2, "s[28:29]") BF_FIX(3, "s[34:35]")
                "s_mov_b64 exec, s[20:21]\n s_mov_b64 s[24:25], 0\n s_mov_b64 s[26:27], 0\n s_mov_b64 s[28:29], 0\n s_mov_b64 s[34:35], 0\n"
                "s_cmp_lg_u32 s22, 0\n s_cbranch_scc1 1b\n"
                "7:\n s_waitcnt lgkmcnt(0)\n"
                : [X0] "+v"(X[0]), [q0] "+v"(q[0]), [n0] "+v"(n1[0]), [acc0] "+v"(acc[0]),
                  [X1] "+v"(X[1]), [q1] "+v"(q[1]), [n1] "+v"(n1[1]), [acc1] "+v"(acc[1]),
                  [X2] "+v"(X[2]), [q2] "+v"(q[2]), [n2] "+v"(n1[2]), [acc2] "+v"(acc[2]),
                  [X3] "+v"(X[3]), [q3] "+v"(q[3]), [n3] "+v"(n1[3]), [acc3] "+v"(acc[3])
                : [L8] "s"(kL << 3)
                : "vcc", "scc", "s20", "s21", "s22", "s24", "s25", "s26", "s27", "s28", "s29", "s30", "s31", "s34", "s35",
                  "v40", "v41", "v42", "v43", "v50", "v51", "v52", "v53", "v60", "v61", "v62", "v63", "v70", "v71", "v72", "v73",
                  "v80", "v81", "v82", "v83", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "memory");
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c) {
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2] = acc[c];
        a.out[((blockIdx.x * blockDim.x + tid) * 4 + c) * 2 + 1] = X[c] >> 3;
    }
}

struct Host {
    uint32_t freq[256], cdf[256]; uint8_t slot_map[4096];
    std::vector<uint2> tab64, tab256; std::vector<uint32_t> tab32;
    std::vector<uint8_t> bodies; std::vector<uint32_t> depth, states;
    std::vector<uint32_t> expect64, expect32, expect256;   // [tile][lane]
    double p0 = 0, p1 = 0, p2 = 0;
};

static void build(Host &h) {
    std::mt19937 rng(1);
    std::normal_distribution<float> nd(0.f, 0.02f);
    std::vector<uint8_t> exps((size_t)kTiles * 2 * kHalf * 32);
    uint64_t count[256] = {0};
    for (auto &e : exps) {
        float f = nd(rng); uint32_t u; memcpy(&u, &f, 4);
        u += 0x7FFF + ((u >> 16) & 1); e = (u >> 23) & 0xFF; count[e]++;
    }
    uint64_t total = exps.size(); uint32_t sum = 0; int arg = 0;
    for (int i = 0; i < 256; ++i) { h.freq[i] = (uint32_t)(count[i] * 4096 / total); if (!h.freq[i]) h.freq[i] = 1; sum += h.freq[i]; if (h.freq[i] > h.freq[arg]) arg = i; }
    h.freq[arg] += 4096 - sum;
    uint32_t c = 0; for (int i = 0; i < 256; ++i) { h.cdf[i] = c; for (uint32_t j = 0; j < h.freq[i]; ++j) h.slot_map[c + j] = i; c += h.freq[i]; }
    h.tab64.resize(4096); h.tab32.resize(4096); h.tab256.resize(4096);
    for (uint32_t s = 0; s < 4096; ++s) { uint32_t y = h.slot_map[s]; h.tab64[s] = make_uint2((h.freq[y] << 3) | (y << 24), (s - h.cdf[y]) << 3); h.tab32[s] = (y << 24) | (h.freq[y] << 12) | (s - h.cdf[y]); h.tab256[s] = make_uint2((h.freq[y] << 8) | (y << 24), (s - h.cdf[y]) << 8); }
    h.bodies.assign((size_t)kTiles * kStr * 64, 0); h.depth.resize(kTiles); h.states.resize(kTiles * 64);
    h.expect64.resize(kTiles * 64); h.expect32.resize(kTiles * 64); h.expect256.resize(kTiles * 64);
    uint64_t n0 = 0, n1 = 0, n2 = 0;
    for (int t = 0; t < kTiles; ++t) {
        std::vector<std::vector<uint8_t>> em(64);
        for (int q = 0; q < 64; ++q) {
            const int hsel = q / 32, col = q % 32; uint32_t x = kL;
            for (int i = kHalf - 1; i >= 0; --i) {
                uint32_t s = exps[(((size_t)t * 2 + hsel) * kHalf + i) * 32 + col], f = h.freq[s];
                while (x >= (f << 12)) { em[q].push_back(x & 0xFF); x >>= 8; }
                x = ((x / f) << 12) + (x % f) + h.cdf[s];
            }
            h.states[t * 64 + q] = x;
        }
        uint32_t d = 0; for (auto &v : em) d = std::max<uint32_t>(d, v.size());
        if (d + 2 > kStr) { printf("body too deep %u\n", d); exit(1); }
        h.depth[t] = d;
        for (int q = 0; q < 64; ++q) { uint32_t pad = d - em[q].size(); for (uint32_t r = pad; r < d; ++r) h.bodies[((size_t)t * kStr + r) * 64 + q] = em[q][r - pad]; }
        for (int q = 0; q < 64; ++q) {   // host decode: checksums and renormalisation statistics
            uint32_t x = h.states[t * 64 + q]; int r = (int)d - 1; uint32_t a64 = 0, a32 = 0, a256 = 0;
            for (int i = 0; i < kHalf; ++i) {
                uint32_t slot = x & 4095, s = h.slot_map[slot];
                if (s != exps[(((size_t)t * 2 + q / 32) * kHalf + i) * 32 + q % 32]) { printf("host decode mismatch\n"); exit(1); }
                a64 += h.tab64[slot].x; a32 += h.tab32[slot]; a256 += h.tab256[slot].x;
                x = h.freq[s] * (x >> 12) + slot - h.cdf[s];
                int k = 0; while (x < kL && r >= 0 && k < 2) { x = (x << 8) | h.bodies[((size_t)t * kStr + r) * 64 + q]; --r; ++k; }
                (k == 0 ? n0 : k == 1 ? n1 : n2)++;
            }
            if (x != kL) { printf("host decode did not end at L\n"); exit(1); }
            h.expect64[t * 64 + q] = a64; h.expect32[t * 64 + q] = a32; h.expect256[t * 64 + q] = a256;
        }
    }
    double n = (double)(n0 + n1 + n2); h.p0 = n0 / n; h.p1 = n1 / n; h.p2 = n2 / n;
}

template <int V> float run(const Host &h, Args a, int waves, int reps, bool check) {
    const size_t ldsb = 32768 + 16 * 64 * kStr;
    CK(hipFuncSetAttribute((const void *)step_kernel<V>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipEvent_t s, e; CK(hipEventCreate(&s)); CK(hipEventCreate(&e));
    hipLaunchKernelGGL(step_kernel<V>, dim3(256), dim3(waves * 64), ldsb, 0, a);
    CK(hipDeviceSynchronize());
    if (check) {
        std::vector<uint32_t> out((size_t)256 * waves * 64 * 2);
        CK(hipMemcpy(out.data(), a.out, out.size() * 4, hipMemcpyDeviceToHost));
        size_t bad = 0;
        for (int b = 0; b < 256; ++b) for (int w = 0; w < waves; ++w) for (int l = 0; l < 64; ++l) {
            const int tile = (b * 16 + w) % kTiles; const size_t i = ((size_t)b * waves * 64 + w * 64 + l) * 2;
            const uint32_t want = (V == 2 ? h.expect32 : V >= 5 ? h.expect256 : h.expect64)[tile * 64 + l] * (uint32_t)a.passes;
            if (out[i] != want || out[i + 1] != kL) ++bad;
        }
        if (bad) printf("  [variant %d, %d waves: %zu wrong lanes]\n", V, waves, bad);
    }
    CK(hipEventRecord(s));
    for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(step_kernel<V>, dim3(256), dim3(waves * 64), ldsb, 0, a);
    CK(hipEventRecord(e)); CK(hipEventSynchronize(e));
    float ms; CK(hipEventElapsedTime(&ms, s, e));
    return ms * 1e6f / reps / (a.passes * kHalf);
}

template <int C, int kKind> float run_cpp(const Host &h, Args a, int waves, int reps) {
    auto kern = kKind == 2 ? bf_kernel<(C == 3) ? 2 : C> : kKind == 1 ? mc_kernel<(C == 2 || C == 4) ? C : 2> : cpp_kernel<C>;
    const size_t ldsb = 32768 + (size_t)waves * C * 64 * kStr;
    if (ldsb > 160 * 1024) return -1.f;
    CK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipEvent_t s, e; CK(hipEventCreate(&s)); CK(hipEventCreate(&e));
    hipLaunchKernelGGL(kern, dim3(256), dim3(waves * 64), ldsb, 0, a);
    CK(hipDeviceSynchronize());
    std::vector<uint32_t> out((size_t)256 * waves * 64 * 8);
    CK(hipMemcpy(out.data(), a.out, out.size() * 4, hipMemcpyDeviceToHost));
    size_t bad = 0;
    for (int b = 0; b < 256; ++b) for (int w = 0; w < waves; ++w) for (int l = 0; l < 64; ++l) for (int c = 0; c < C; ++c) {
        const int tile = ((b * 16 + w) * C + c) % kTiles; const size_t i = ((((size_t)b * waves * 64 + w * 64 + l) * 4) + c) * 2;
        if (out[i] != h.expect64[tile * 64 + l] * (uint32_t)a.passes || out[i + 1] != kL) ++bad;
    }
    if (bad) printf("  [cpp C=%d, %d waves: %zu wrong]\n", C, waves, bad);
    CK(hipEventRecord(s));
    for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, dim3(256), dim3(waves * 64), ldsb, 0, a);
    CK(hipEventRecord(e)); CK(hipEventSynchronize(e));
    float ms; CK(hipEventElapsedTime(&ms, s, e));
    return ms * 1e6f / reps / (a.passes * kHalf) / (waves * C);   // ns of a CU per wavefront-step
}

template <int K> float run_lds(uint32_t *out, int waves) {
    CK(hipFuncSetAttribute((const void *)lds_kernel<K>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipEvent_t s, e; CK(hipEventCreate(&s)); CK(hipEventCreate(&e));
    const int iters = 4096;
    hipLaunchKernelGGL(lds_kernel<K>, dim3(256), dim3(waves * 64), 65536, 0, out, iters);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(s));
    for (int i = 0; i < 3; ++i) hipLaunchKernelGGL(lds_kernel<K>, dim3(256), dim3(waves * 64), 65536, 0, out, iters);
    CK(hipEventRecord(e)); CK(hipEventSynchronize(e));
    float ms; CK(hipEventElapsedTime(&ms, s, e));
    return ms * 1e6f / 3 / (iters * 8.0f) / waves;   // ns of a CU per wavefront-wide read
}

int main() {
    Host h; build(h);
    printf("renormalisation bytes per step: 0: %.4f  1: %.4f  2: %.5f\n", h.p0, h.p1, h.p2);
    Args a; a.passes = 16;
    uint2 *t64, *t256; uint32_t *t32; uint8_t *bod; uint32_t *dep, *sta, *out;
    CK(hipMalloc(&t64, 32768)); CK(hipMalloc(&t256, 32768)); CK(hipMalloc(&t32, 16384)); CK(hipMalloc(&bod, h.bodies.size())); CK(hipMalloc(&dep, kTiles * 4));
    CK(hipMalloc(&sta, kTiles * 64 * 4)); CK(hipMalloc(&out, 256 * 1024 * 8 * 4));
    CK(hipMemcpy(t64, h.tab64.data(), 32768, hipMemcpyHostToDevice)); CK(hipMemcpy(t256, h.tab256.data(), 32768, hipMemcpyHostToDevice)); CK(hipMemcpy(t32, h.tab32.data(), 16384, hipMemcpyHostToDevice));
    CK(hipMemcpy(bod, h.bodies.data(), h.bodies.size(), hipMemcpyHostToDevice)); CK(hipMemcpy(dep, h.depth.data(), kTiles * 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(sta, h.states.data(), kTiles * 64 * 4, hipMemcpyHostToDevice));
    a.tab64 = t64; a.tab32 = t32; a.tab256 = t256; a.bodies = bod; a.depth = dep; a.states = sta; a.out = out;
    printf("ns of a CU per wavefront-wide LDS read (16 / 8 wavefronts per CU)\n");
    printf("  b64 random %.2f %.2f | b32 random %.2f %.2f | u8 lane columns %.2f %.2f | b64 one address %.2f %.2f\n",
           run_lds<0>(out, 16), run_lds<0>(out, 8), run_lds<1>(out, 16), run_lds<1>(out, 8), run_lds<2>(out, 16), run_lds<2>(out, 8),
           run_lds<3>(out, 16), run_lds<3>(out, 8));
    fflush(stdout);
    a.passes = 32;
    printf("ns of a CU per wavefront-step\n");
    printf("waves/CU  old-3-LDS  masked(shipping)  x256-branch-free  x256-masked  x256-bf-deferred | masked 2 chains | branch-free(old) 1 chain\n");
    for (int w : {1, 4, 8, 12, 14, 16}) {
        float t0 = run<0>(h, a, w, 5, true) / w, t1 = run<1>(h, a, w, 5, true) / w, t5 = run<5>(h, a, w, 5, true) / w, t6 = run<6>(h, a, w, 5, true) / w, t7 = run<7>(h, a, w, 5, true) / w;
        printf("%8d  %6.2f %6.2f %6.2f %6.2f %6.2f | %6.2f | %6.2f\n", w, t0, t1, t5, t6, t7, run_cpp<2, 1>(h, a, w, 5), run_cpp<1, 2>(h, a, w, 5));
        fflush(stdout);
    }
    return 0;
}
