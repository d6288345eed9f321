// Fused decompress + GEMV/GEMM and the split-K reduction (gfx950).
//
// out[M,N] = x[M,K] * W[K,N] (+ bias), W stored as rANS-coded exponent plane + raw
// sign|mantissa plane; W is never materialised.  Replaces fused_rans_linear_triton and its
// kernel fused_rans_matmul_kernel_ilp2_splitk (comp_inference/linear_triton.py:229-552) and
// the torch.sum split-K reduction (comp_inference/linear_triton.py:303-314).
//
// Mapping for the default 32-column tile: one wavefront per tile; lanes 0..31 decode the
// top-half streams of the tile's 32 columns, lanes 32..63 the bottom-half streams.  After 8
// decode steps lane l holds 8 consecutive-k bf16 weights of column l%32 -- which is exactly
// the A-operand fragment of v_mfma_f32_32x32x16_bf16 (A = W^T tile, 32 columns x 16 k, where
// k 0..7 are the 8 top-half rows and k 8..15 the 8 bottom-half rows).  The B operand is the
// matching slice of x for up to 32 rows of M, loaded straight from global memory.  One MFMA per
// 8 decode steps does the whole contraction for any M <= 32, so the VALU only decodes.
//
// A workgroup is kw x nw waves: kw k-tiles of nw neighbouring column tiles.  The kw partial
// accumulators are summed through LDS in a fixed order (deterministic); if one workgroup spans
// all of K the result is written as bf16 directly, otherwise fp32 partials go to a workspace and
// splitk_reduce_kernel sums them in index order.
#include "ci_common.h"
#include "rans_device.h"
#include "fast_tile.h"

namespace ci {

constexpr int kLinMaxWaves = 8;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct LinearArgs {
    const uint16_t *x;
    uint32_t M, K, N, x_stride;
    const uint8_t *stream;
    uint64_t stream_len;
    const uint32_t *states;
    const uint32_t *tables;
    const uint8_t *slot_map;
    const uint32_t *tile_offsets;
    const uint32_t *tile_max_lens;
    const uint32_t *stream_offsets;  // dense layout
    const uint32_t *stream_sizes;    // dense layout
    const uint8_t *man_tiled;
    const uint16_t *bias;
    float *partial;   // [P][M][N] when P > 1
    uint16_t *out;    // [M][N]
    uint32_t out_stride;
    uint32_t th, tw, tiles_n, tiles_k, kw, nw, P;
    int fast_ok;  // x rows may be read with 16-byte loads at 32-bit offsets, sign|mantissa plane dword aligned
    // x rearranged so that one MFMA operand load reads whole cache lines: fragment (group g of 32 rows,
    // block kb of 8 k, row mm) = 16 bytes at ((g * K/8 + kb) * 32 + mm) * 16, rows >= M zero; or null
    const uint16_t *xf;
    // Verification aid: when set, the weights are read from this plain bf16 [K, N] matrix instead of
    // being decoded (every tile takes the guarded path, which issues the same MFMA sequence as the
    // hand-scheduled one); none of the compressed operands is touched.
    const uint16_t *dense_w;
    // Decoder checkpoints (ci_build_checkpoints_ilp2) and the number of segments per stream they cut, or
    // null / 1: with them the resident kernel gives every (tile, segment) its own wavefront.
    const uint2 *ckpt;
    uint32_t segs;
    // The 32 KB slot table of the scaled state (build_slot_table_x8) kept beside the weight, or null: then
    // every workgroup builds it from tables and slot_map.
    const uint2 *slot_table;
    uint32_t rounds;  // fused_linear32_seg_kernel: items of a job per wavefront
    bool all_fast;    // every item of the weight takes the hand-scheduled loop (known from the descriptor)
    uint32_t wait_limit;  // looks a wavefront takes at another wavefront's flag before it gives up (see g_device_status)
};

// What a kernel could not do and did not hang over, one bit per kind (ci_device_status reads and clears it):
// a wavefront that waits for another one inside a kernel looks at the flag at most LinearArgs::wait_limit times, then
// records CI_STATUS_WAIT_GAVE_UP here and goes on, so that a slip in a hand-over shows as an error code and wrong
// sums, never as a kernel that does not end.
static __device__ uint32_t g_device_status;

// x [M, K] -> the fragment order described at LinearArgs::xf.  In a plain row-major x the 64 lanes of
// one operand load touch 64 different cache lines (16 bytes of each); with many rows that traffic, not
// the decoding, bounds the kernel.
__global__ __launch_bounds__(256) void x_fragments_kernel(const uint16_t *__restrict__ x, uint32_t M, uint32_t K,
                                                          uint32_t x_stride, u32x4 *__restrict__ xf,
                                                          uint32_t total) {
    const uint32_t e = blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const uint32_t kbs = K / 8, mm = e % 32, kb = (e / 32) % kbs, g = e / (32 * kbs), row = g * 32 + mm;
    u32x4 v = (u32x4){0, 0, 0, 0};
    if (row < M) v = *reinterpret_cast<const u32x4 *>(x + (size_t)row * x_stride + (size_t)kb * 8);
    xf[e] = v;
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// torch semantics of `out_bf16 += bias_bf16`: add in fp32, round once.
__device__ __forceinline__ uint16_t finish_bf16(float acc, const uint16_t *bias, uint32_t n) {
    uint16_t r = f32_to_bf16_rne(acc);
    if (bias) r = f32_to_bf16_rne(bf16_to_f32(r) + bf16_to_f32(bias[n]));
    return r;
}

// Two decoded symbols (top bytes of w0, w1) + two sign|mantissa bytes -> two bf16 in one dword
// (row of w0 in the low half).  The sign|mantissa bytes are byte `b` of m0 / m1, chosen by
// man_sel = 0x04040000 + b * 0x01010101.
__device__ __forceinline__ uint32_t pack_bf16_pair(uint32_t w0, uint32_t w1, uint32_t m0, uint32_t m1,
                                                   uint32_t man_sel = 0x04040000u) {
    const uint32_t e = __builtin_amdgcn_perm(w1, w0, 0x070C030Cu) >> 1;  // s1 << 23 | s0 << 7
    const uint32_t mm = __builtin_amdgcn_perm(m1, m0, man_sel);           // [m1 m1 m0 m0]
    return (e & 0x7F807F80u) | (mm & 0x807F807Fu);
}

// General path: ragged tiles (rows >= K, columns >= N), unaligned x, odd block counts, or a tile
// body too deep for the staging area.  Same arithmetic on the scaled state, bytes read where they
// lie in global memory, every access guarded.
// wd: null, or this lane's column of a plain bf16 weight at row k0 (row stride wd_stride elements).
__device__ __forceinline__ void linear_tile_guarded(GlobalBytes &src, uint32_t X, const uint2 *tab, uint32_t K,
                                                    uint32_t half, uint32_t my_steps, const uint8_t *man,
                                                    const uint16_t *xrow, bool m_ok, uint32_t k0, f32x16 &acc,
                                                    const uint16_t *wd = nullptr, uint32_t wd_stride = 0) {
    for (uint32_t i = 0; i < half; i += 8) {
        u32x4 xv = (u32x4){0, 0, 0, 0};
        if (m_ok) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t k = k0 + i + j;
                const uint32_t v = k < K ? xrow[i + j] : 0u;
                xv[j / 2] |= v << (16 * (j & 1));
            }
        }
        uint32_t mb[8], w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            mb[j] = 0;
            w[j] = 0;
            if (!wd && i + j < my_steps) {
                mb[j] = man[(size_t)(i + j) * 32];
                w[j] = decode_symbol_scaled(X, tab);
                src.renorm_scaled(X);
                src.renorm_scaled(X);
            }
        }
        u32x4 wv;
        if (wd) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const uint32_t lo = i + 2 * p < my_steps ? wd[(size_t)(i + 2 * p) * wd_stride] : 0u;
                const uint32_t hi = i + 2 * p + 1 < my_steps ? wd[(size_t)(i + 2 * p + 1) * wd_stride] : 0u;
                wv[p] = lo | (hi << 16);
            }
        } else {
#pragma unroll
            for (int p = 0; p < 4; ++p) wv[p] = pack_bf16_pair(w[2 * p], w[2 * p + 1], mb[2 * p], mb[2 * p + 1]);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wv), __builtin_bit_cast(bf16x8, xv),
                                                      acc, 0, 0, 0);
    }
}

// grid: (ceil(tiles_n / nw), P, ceil(M / (32 * MB)))   block: kw * nw waves
// MB = 32-row groups of x per pass over the weight: 1, or 2 (M > 32: the weight is decoded once per
// 64 rows and feeds two accumulators).
template <int MB>
__global__ __launch_bounds__(kLinMaxWaves *kWave) void fused_linear32_kernel(LinearArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint2 *tab = reinterpret_cast<uint2 *>(lds);
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int nthreads = blockDim.x;
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kFastStageBytes;

    const uint32_t kidx = wave % a.kw, nidx = wave / a.kw;
    const uint32_t tk = blockIdx.y * a.kw + kidx, tn = blockIdx.x * a.nw + nidx;
    const bool have_tile = tk < a.tiles_k && tn < a.tiles_n;
    const uint32_t tile = tk * a.tiles_n + tn;
    const uint32_t half = a.th / 2, hsel = lane / 32, c = lane % 32;
    const uint32_t col0 = tn * 32, k0 = tk * a.th + hsel * half;
    uint32_t depth = 0, my_steps = 0, state = 0;
    uint64_t base = 0;
    bool fast = false;
    StageRegs body;
    if (have_tile && a.dense_w) {
        if (col0 + c < a.N && k0 < a.K) my_steps = min(half, a.K - k0);
    } else if (have_tile) {
        base = a.tile_offsets[tile];
        depth = a.tile_max_lens[tile];
        state = a.states[(size_t)tile * 64 + lane];
        if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;
        if (col0 + c < a.N && k0 < a.K) my_steps = min(half, a.K - k0);
        const bool full = __builtin_amdgcn_ballot_w64(my_steps != half) == 0;
        // the hand-scheduled loop wants: a full tile, a body that fits one lane stride, an even
        // number of 8-row blocks, 16-byte readable x rows and a dword-aligned sign|mantissa plane
        fast = full && a.fast_ok && depth >= 2 && depth < kFastStride && half % 16 == 0 &&
               (uint32_t)(uintptr_t)tab == 0;  // (depth is 0 in a plain-weight run)
        if (fast) stage_fetch(body, a.stream + base, 0, depth, lane);
    }
    if (!a.dense_w) build_slot_table_x8(tab, a.tables, a.slot_map, tid, nthreads);  // runs under the body loads
    if (fast) {
        stage_commit(body, stage, 0, depth, lane);
        for (int grp = 1; grp < kStageGroups; ++grp)
            if ((uint32_t)grp * 128 < depth) {
                stage_fetch(body, a.stream + base, grp * 128, depth, lane);
                stage_commit(body, stage, grp * 128, depth, lane);
            }
    }
    __syncthreads();

    const uint32_t m = blockIdx.z * (32 * MB) + c;  // row of x this lane feeds to the (first) MFMA
    const bool m_ok = m < a.M, m2_ok = MB == 2 && m + 32 < a.M;
    f32x16 acc, acc2;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = acc2[v] = 0.f;

    if (have_tile) {
        const uint32_t xrow_elems = (m_ok ? m : 0) * a.x_stride + k0;  // rows past M re-read row 0: their
                                                                       // accumulator columns are never stored
        const uint32_t xrow2_elems = (m2_ok ? m + 32 : 0) * a.x_stride + k0;
        const size_t man_tile = (size_t)tile * a.th * 32;
        if (fast) {
            FastLane st;
            st.init(stage, depth, lane, state);
            const uint64_t mbase = reinterpret_cast<uint64_t>(a.man_tiled + man_tile);
            // readfirstlane returns a signed int: widen through uint32_t, not by sign extension
            const uint32_t mb_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(mbase >> 32));
            const uint32_t mb_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)mbase);
            const uint64_t mb_u = ((uint64_t)mb_hi << 32) | (uint64_t)mb_lo;
            const uint32_t moff = hsel * half * 32 + (c & ~3u);
            const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
            uint64_t xb = reinterpret_cast<uint64_t>(a.x);
            uint32_t xo = xrow_elems * 2u, xo2 = xrow2_elems * 2u, xstep = 16;
            if (a.xf) {  // fragment order: this lane's row slot c of group g, block k0 / 8 onwards
                const uint32_t kbs = a.K / 8, g = blockIdx.z * MB;
                xb = reinterpret_cast<uint64_t>(a.xf);
                xo = ((g * kbs + k0 / 8) * 32 + c) * 16;
                xo2 = xo + kbs * 32 * 16;
                xstep = 32 * 16;
            }
            if (MB == 2)
                linear_tile_asm2(st, acc, acc2, mb_u, moff, xb, xo, xo2, xstep, man_sel, half / 8);
            else
                linear_tile_asm(st, acc, mb_u, moff, xb, xo, xstep, man_sel, half / 8);
        } else {
            const uint8_t *man = a.man_tiled + man_tile + (size_t)hsel * half * 32 + c;
            // only rows below my_steps are read, and that is 0 for a lane outside the matrix
            const uint16_t *wd = a.dense_w ? a.dense_w + (size_t)k0 * a.N + col0 + c : nullptr;
            GlobalBytes src;
            src.init(a.stream + base, depth, 64, lane);
            linear_tile_guarded(src, state << 3, tab, a.K, half, my_steps, man, a.x + xrow_elems, m_ok, k0, acc,
                                wd, a.N);
            if (MB == 2) {  // the guarded path simply walks the tile again for the second group of rows
                src.init(a.stream + base, depth, 64, lane);
                linear_tile_guarded(src, state << 3, tab, a.K, half, my_steps, man, a.x + xrow2_elems, m2_ok, k0, acc2,
                                    wd, a.N);
            }
        }
    }

    // Sum the kw accumulators of each column tile in k order.  The staging area is free now;
    // every wave stores its fragment(s) as [v][lane] floats (4 KB each).
    __syncthreads();
    float *red = reinterpret_cast<float *>(lds + kSlotTableBytes);
    const uint32_t frag = 16 * kWave;
#pragma unroll
    for (int g = 0; g < MB; ++g) {
        const f32x16 &part = g ? acc2 : acc;
        const uint32_t mg = m + 32 * g;
        if (g) __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v) red[(size_t)wave * frag + v * kWave + lane] = part[v];
        __syncthreads();
        if (kidx == 0 && tn < a.tiles_n) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float s = 0.f;
                for (uint32_t kk = 0; kk < a.kw; ++kk) s += red[(size_t)(nidx * a.kw + kk) * frag + v * kWave + lane];
                // MFMA 32x32 result layout: register v of lane l is row (v/4)*8 + (l/32)*4 + v%4
                // (= column of the tile), column l%32 (= row m of x)
                const uint32_t n = tn * 32 + (v / 4) * 8 + hsel * 4 + (v % 4);
                if (mg < a.M && n < a.N) {
                    if (a.P == 1)
                        a.out[(size_t)mg * a.out_stride + n] = finish_bf16(s, a.bias, n);
                    else
                        a.partial[((size_t)blockIdx.y * a.M + mg) * a.N + n] = s;
                }
            }
        }
    }
}

// ---- more than 64 rows of x in one pass over the weight ---------------------------------------------------
// The same decomposition as fused_linear32_kernel (a wavefront per tile, kw k-tiles of nw column tiles per
// workgroup, the kw accumulators of a column tile added through LDS in k order), with MB = 4 or 8 groups of 32
// rows of x per pass: a tile is decoded once, its eight-row weight fragments stay in registers, and every
// fragment goes into MB matrix instructions, one per group of rows, against the x fragments of the copy in
// fragment order (LinearArgs::xf, which this kernel needs).  The decode cost is then paid once per 128 or 256
// rows instead of once per 64.  Every row of x still sees the same sequence of matrix instructions and the same
// sums as in fused_linear32_kernel, so the results are bit-identical to it.
// grid: (ceil(tiles_n / nw), P, ceil(M / (32 * MB)))   block: kw * nw waves
template <int MB>
__device__ __forceinline__ void linear_tile_wide(FastLane &st, f32x16 (&acc)[MB], const uint32_t *__restrict__ mrow,
                                                 const u32x4 *__restrict__ xrow, uint32_t group_stride,
                                                 uint32_t man_sel, uint32_t nblk) {
    // mrow: the aligned dword holding this lane's sign|mantissa byte of the tile half's first row (+ 8 dwords per
    // row); xrow: this lane's 16 bytes of the first block's fragment of the pass's first group (+ 32 per block,
    // + group_stride per group).  The next block's operands are loaded while this one decodes.
    uint32_t mcur[8], mnext[8];
    u32x4 xcur[MB], xnext[MB];
#pragma unroll
    for (int r = 0; r < 8; ++r) mcur[r] = mrow[r * 8];
#pragma unroll
    for (int g = 0; g < MB; ++g) xcur[g] = xrow[(size_t)g * group_stride];
    for (uint32_t blk = 0; blk < nblk; ++blk) {
        const uint32_t nb = blk + 1 < nblk ? blk + 1 : blk;  // (the last block re-reads its own: stays inside the tile)
#pragma unroll
        for (int r = 0; r < 8; ++r) mnext[r] = mrow[(size_t)nb * 64 + r * 8];
#pragma unroll
        for (int g = 0; g < MB; ++g) xnext[g] = xrow[(size_t)nb * 32 + (size_t)g * group_stride];
        uint32_t w[4];
        decode8_weights_asm(st, mcur, man_sel, w);
        // (the statement's last instruction but one writes w[3]: a matrix instruction may read a register a vector
        // instruction wrote no sooner than two wait states later, and the compiler does not see inside the
        // statement; w[3] passes through the wait, so whatever reads it comes after)
        asm volatile("s_nop 1" : "+v"(w[3]));
        const u32x4 wv = {w[0], w[1], w[2], w[3]};
#pragma unroll
        for (int g = 0; g < MB; ++g)
            acc[g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, wv),
                                                             __builtin_bit_cast(bf16x8, xcur[g]), acc[g], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 8; ++r) mcur[r] = mnext[r];
#pragma unroll
        for (int g = 0; g < MB; ++g) xcur[g] = xnext[g];
    }
}

template <int MB>
__global__ __launch_bounds__(kLinMaxWaves *kWave) void fused_linear32_wide_kernel(LinearArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint2 *tab = reinterpret_cast<uint2 *>(lds);
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int nthreads = blockDim.x;
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kFastStageBytes;

    const uint32_t kidx = wave % a.kw, nidx = wave / a.kw;
    const uint32_t tk = blockIdx.y * a.kw + kidx, tn = blockIdx.x * a.nw + nidx;
    const bool have_tile = tk < a.tiles_k && tn < a.tiles_n;
    const uint32_t tile = tk * a.tiles_n + tn;
    const uint32_t half = a.th / 2, hsel = lane / 32, c = lane % 32;
    const uint32_t col0 = tn * 32, k0 = tk * a.th + hsel * half;
    uint32_t depth = 0, my_steps = 0, state = 0;
    uint64_t base = 0;
    bool fast = false;
    StageRegs body;
    if (have_tile) {
        base = a.tile_offsets[tile];
        depth = a.tile_max_lens[tile];
        state = a.states[(size_t)tile * 64 + lane];
        if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;
        if (col0 + c < a.N && k0 < a.K) my_steps = min(half, a.K - k0);
        const bool full = __builtin_amdgcn_ballot_w64(my_steps != half) == 0;
        // the same conditions as fused_linear32_kernel's hand-scheduled loop (a tile takes the same path in both)
        fast = full && a.fast_ok && depth >= 2 && depth < kFastStride && half % 16 == 0 && (uint32_t)(uintptr_t)tab == 0;
        if (fast) stage_fetch(body, a.stream + base, 0, depth, lane);
    }
    build_slot_table_x8(tab, a.tables, a.slot_map, tid, nthreads);  // runs under the body loads
    if (fast) {
        stage_commit(body, stage, 0, depth, lane);
        for (int grp = 1; grp < kStageGroups; ++grp)
            if ((uint32_t)grp * 128 < depth) {
                stage_fetch(body, a.stream + base, grp * 128, depth, lane);
                stage_commit(body, stage, grp * 128, depth, lane);
            }
    }
    __syncthreads();

    const uint32_t g0 = blockIdx.z * MB;  // first 32-row group of this pass
    f32x16 acc[MB];
#pragma unroll
    for (int g = 0; g < MB; ++g)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[g][v] = 0.f;

    if (have_tile) {
        const size_t man_tile = (size_t)tile * a.th * 32;
        if (fast) {
            FastLane st;
            st.init(stage, depth, lane, state);
            // (the fragment copy holds whole passes: its groups past the last row of x are zero)
            const uint32_t kbs = a.K / 8;
            const u32x4 *xrow = reinterpret_cast<const u32x4 *>(a.xf) + ((size_t)g0 * kbs + k0 / 8) * 32 + c;
            const uint32_t *mrow =
                reinterpret_cast<const uint32_t *>(a.man_tiled + man_tile + (size_t)hsel * half * 32 + (c & ~3u));
            const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
            linear_tile_wide<MB>(st, acc, mrow, xrow, kbs * 32, man_sel, half / 8);
        } else {
            const uint8_t *man = a.man_tiled + man_tile + (size_t)hsel * half * 32 + c;
#pragma unroll
            for (int g = 0; g < MB; ++g) {  // the guarded path walks the tile again for every group of rows
                const uint32_t m = (g0 + g) * 32 + c;
                const bool m_ok = m < a.M;
                GlobalBytes src;
                src.init(a.stream + base, depth, 64, lane);
                linear_tile_guarded(src, state << 3, tab, a.K, half, my_steps, man,
                                    a.x + (size_t)(m_ok ? m : 0) * a.x_stride + k0, m_ok, k0, acc[g]);
            }
        }
    }

    // Sum the kw accumulators of each column tile in k order (as in fused_linear32_kernel).
    __syncthreads();
    float *red = reinterpret_cast<float *>(lds + kSlotTableBytes);
    const uint32_t frag = 16 * kWave;
#pragma unroll
    for (int g = 0; g < MB; ++g) {
        const uint32_t mg = (g0 + g) * 32 + c;
        if (g) __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v) red[(size_t)wave * frag + v * kWave + lane] = acc[g][v];
        __syncthreads();
        if (kidx == 0 && tn < a.tiles_n) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float s = 0.f;
                for (uint32_t kk = 0; kk < a.kw; ++kk) s += red[(size_t)(nidx * a.kw + kk) * frag + v * kWave + lane];
                const uint32_t n = tn * 32 + (v / 4) * 8 + hsel * 4 + (v % 4);
                if (mg < a.M && n < a.N) {
                    if (a.P == 1)
                        a.out[(size_t)mg * a.out_stride + n] = finish_bf16(s, a.bias, n);
                    else
                        a.partial[((size_t)blockIdx.y * a.M + mg) * a.N + n] = s;
                }
            }
        }
    }
}

// The same tile work with workgroups resident for the launch (fast_tile.h): wavefront w of workgroup j
// takes the items j + (w + n i) * gridDim.x and writes its 32-column partial product to the fp32 workspace
// [tiles_k * segs][M][N], which the reduction kernel sums in k order.  For weights with more tiles than
// the chip holds at once (fused gate/up projections), where the 8-wavefront workgroups of the kernel
// above would run in two full rounds -- and for weights with so few tiles that their th/2-step chains,
// not the chip, bound the time: with decoder checkpoints every stream is cut into `segs` segments
// and an item is one segment of the 64 streams of a tile.  M <= 32 * MB.
//
// Item vk * tiles_n + tn, vk = tk * segs + seg: rows [seg, seg + 1) * th / (2 segs) of both halves of tile
// (tk, tn).  A segment's bytes are the rows between its own checkpoint and the next one's, about
// depth / segs of them per lane plus the spread between lanes; only that window of the body is staged.
// kKeep: the item's products are added to acc / acc2 and stay there (the caller owns the sum); otherwise the
// item starts from zero and writes its own partial sums to the workspace.
template <int MB, uint32_t kStride, bool kKeep = false>
__device__ __forceinline__ void linear_one_item(const LinearArgs &a, uint32_t vk, uint32_t tn, const uint2 *tab,
                                                uint8_t *stage, int lane, f32x16 &acc, f32x16 &acc2) {
    const uint32_t tk = vk / a.segs, seg = vk % a.segs, tile = tk * a.tiles_n + tn;
    const uint32_t half = a.th / 2, seglen = half / a.segs, hsel = lane / 32, c = lane % 32;
    const uint32_t col0 = tn * 32, k0 = tk * a.th + hsel * half + seg * seglen;
    const uint64_t base = a.dense_w ? 0 : a.tile_offsets[tile];
    uint32_t depth = a.dense_w ? 0 : a.tile_max_lens[tile];
    if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;
    // decoder state and row of the next unread byte at the first row of the segment, and at its end
    uint32_t state = 0;
    int32_t row = (int32_t)depth - 1, row_end = -1;
    if (!a.dense_w) {
        const uint2 *ck = a.ckpt + ((size_t)tile * (a.segs - 1)) * 64 + lane;  // (only read when segs > 1)
        if (seg == 0) {
            state = a.states[(size_t)tile * 64 + lane];
        } else {
            const uint2 v = ck[(size_t)(seg - 1) * 64];
            state = v.x;
            row = min((int32_t)v.y, (int32_t)depth - 1);
        }
        if (seg + 1 < a.segs) row_end = min((int32_t)ck[(size_t)seg * 64].y, row);
    }
    uint32_t my_steps = 0;
    if (col0 + c < a.N && k0 < a.K) my_steps = min(seglen, a.K - k0);
    const bool full = __builtin_amdgcn_ballot_w64(my_steps != seglen) == 0;
    // rows of the body this item can touch: from the lowest end row (less the two prefetched bytes) to the
    // highest start row
    const int32_t lo = max(wave_min_i32(row_end) - 1, 0), hi = wave_max_i32(row);
    const uint32_t window = hi >= lo ? (uint32_t)(hi - lo + 1) : 0u;
    // (kStride == 0: a caller without a transposed staging area; every item takes the guarded path)
    const bool fast = kStride != 0 && full && a.fast_ok && window >= 2 && window < kStride && seglen % 16 == 0 &&
                      (uint32_t)(uintptr_t)tab == 0 && !a.dense_w;
    const uint32_t m = c;  // row of x this lane feeds to the (first) MFMA
    const bool m_ok = m < a.M, m2_ok = MB == 2 && m + 32 < a.M;
    if (!kKeep) {
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = acc2[v] = 0.f;
    }
    const uint32_t xrow_elems = (m_ok ? m : 0) * a.x_stride + k0;
    const uint32_t xrow2_elems = (m2_ok ? m + 32 : 0) * a.x_stride + k0;
    const size_t man_tile = (size_t)tile * a.th * 32;
    if (fast) {
        if constexpr (kStride != 0) {
        stage_body<kStride>(stage, a.stream + base + (size_t)lo * 64, window, lane);
        FastLane st;
        st.init_at<kStride>(stage, row - lo + 1, lane, state);
        const uint64_t mbase = reinterpret_cast<uint64_t>(a.man_tiled + man_tile);
        // readfirstlane returns a signed int: widen through uint32_t, not by sign extension
        const uint32_t mb_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(mbase >> 32));
        const uint32_t mb_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)mbase);
        const uint64_t mb_u = ((uint64_t)mb_hi << 32) | (uint64_t)mb_lo;
        const uint32_t moff = (hsel * half + seg * seglen) * 32 + (c & ~3u);
        const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
        uint64_t xb = reinterpret_cast<uint64_t>(a.x);
        uint32_t xo = xrow_elems * 2u, xo2 = xrow2_elems * 2u, xstep = 16;
        if (a.xf) {
            const uint32_t kbs = a.K / 8;
            xb = reinterpret_cast<uint64_t>(a.xf);
            xo = ((k0 / 8) * 32 + c) * 16;
            xo2 = xo + kbs * 32 * 16;
            xstep = 32 * 16;
        }
        if (MB == 2)
            linear_tile_asm2(st, acc, acc2, mb_u, moff, xb, xo, xo2, xstep, man_sel, seglen / 8);
        else
            linear_tile_asm(st, acc, mb_u, moff, xb, xo, xstep, man_sel, seglen / 8);
        }
    } else {
        const uint8_t *man = a.man_tiled + man_tile + (size_t)(hsel * half + seg * seglen) * 32 + c;
        const uint16_t *wd = a.dense_w ? a.dense_w + (size_t)k0 * a.N + col0 + c : nullptr;
        GlobalBytes src;
        src.init(a.stream + base, (uint32_t)(row + 1), 64, lane);
        linear_tile_guarded(src, state << 3, tab, a.K, seglen, my_steps, man, a.x + xrow_elems, m_ok, k0, acc, wd, a.N);
        if (MB == 2) {
            src.init(a.stream + base, (uint32_t)(row + 1), 64, lane);
            linear_tile_guarded(src, state << 3, tab, a.K, seglen, my_steps, man, a.x + xrow2_elems, m2_ok, k0, acc2, wd,
                                a.N);
        }
    }
    if (kKeep) return;
    // MFMA 32x32 result layout: register v of lane l is row (v/4)*8 + (l/32)*4 + v%4 (= column of
    // the tile), column l%32 (= row m of x)
#pragma unroll
    for (int g = 0; g < MB; ++g) {
        const f32x16 &part = g ? acc2 : acc;
        const uint32_t mg = m + 32 * g;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t n = col0 + (v / 4) * 8 + hsel * 4 + (v % 4);
            if (mg < a.M && n < a.N) a.partial[((size_t)vk * a.M + mg) * a.N + n] = part[v];
        }
    }
}

template <int MB, int kWaves, uint32_t kStride>
__device__ __forceinline__ void linear_wave_tiles(const LinearArgs &a, const uint2 *tab, uint8_t *lds, int wave, int lane) {
    const uint64_t num_items = (uint64_t)a.tiles_k * a.segs * a.tiles_n;
    // Items of this workgroup, the rounds they take on kWaves wavefronts, and the fewest wavefronts that do
    // them in as many rounds: 12 items run as 6 + 6, not 11 + 1 (a round lasts as long as a full one however
    // few wavefronts take part, and fewer wavefronts at a time step faster).
    const uint32_t mine = blockIdx.x < num_items ? (uint32_t)((num_items - blockIdx.x + gridDim.x - 1) / gridDim.x) : 0u;
    const uint32_t rounds = (mine + kWaves - 1) / kWaves;
    const uint32_t active = rounds ? (mine + rounds - 1) / rounds : 0u;
    if ((uint32_t)wave >= active) return;
    uint8_t *stage = persist_stage<kWaves, kStride>(lds, wave);
    f32x16 acc, acc2;
    for (uint64_t item = (uint64_t)wave * gridDim.x + blockIdx.x; item < num_items; item += (uint64_t)active * gridDim.x)
        linear_one_item<MB, kStride>(a, (uint32_t)(item / a.tiles_n), (uint32_t)(item % a.tiles_n), tab, stage, lane, acc,
                                     acc2);
}

template <int MB>
__global__ __launch_bounds__(kPersistWaves *kWave) void fused_linear32_resident_kernel(LinearArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    // (a plain-weight run has no table to build; which wavefront takes which tile does not change a tile's sum)
    uint32_t cls = 0;
    if (!a.dense_w && a.segs <= 1) {
        cls = persist_prologue(lds, a.tables, a.slot_map, a.tile_max_lens, a.tiles_k * a.tiles_n, blockIdx.x, gridDim.x);
    } else if (!a.dense_w) {
        // a segment's window is about its share of the body plus the spread between the lanes; an item
        // whose window turns out larger than the class allows takes the guarded path
        uint32_t deepest = 0;
        for (uint32_t t = threadIdx.x; t < a.tiles_k * a.tiles_n; t += kPersistWaves * kWave)
            deepest = max(deepest, a.tile_max_lens[t]);
        cls = persist_classify(lds, a.tables, a.slot_map, deepest / a.segs + 40);
    }
    if (cls == 2u)
        linear_wave_tiles<MB, 8, kDepthDeep>(a, tab, lds, wave, lane);
    else if (cls == 1u)
        linear_wave_tiles<MB, 10, kDepthMedium>(a, tab, lds, wave, lane);
    else if (cls == 0u)
        linear_wave_tiles<MB, 11, kDepthShallow>(a, tab, lds, wave, lane);
    else
        linear_wave_tiles<MB, 12, kDepthTiny>(a, tab, lds, wave, lane);
}

// ---- sixteen wavefronts per CU on short items ---------------------------------------------------
// The decode step is bound by how many wavefronts a CU keeps in flight (a step is a chain of dependent
// instructions; four wavefronts per SIMD are what hides it), and sixteen wavefronts leave each 128
// VGPRs and, next to the 32 KB slot table, 7 KB of LDS.  So this kernel takes items whose stream bytes
// are few: a segment of the 64 streams of a tile (decoder checkpoints), or a whole tile when tiles are
// low.  What such an item reads of the tile body is a window of at most kWinRows rows, staged as it lies
// in memory (row r of the window at 64 r, one byte per lane: the stream pointer of a lane moves by 64),
// which takes no lane exchanges and no VALU work.  A wavefront walks its list of items with what an item
// needs from memory asked for ahead: the checkpoints of the item after the next are requested, and the
// cache lines of the next item's window and first sign|mantissa rows are touched, before the current
// item's loop starts, so that between two items a wavefront waits for cache hits, not for HBM.
constexpr int kSegWaves = 16;
constexpr uint32_t kWinRows = kPairWinRows;
constexpr uint32_t kWinBytes = kWinRows * 64;
// Behind the windows: for up to kSmallM rows of x, the sums a wavefront hands over at the end of a job (32
// tile columns per row of x), and two words of bookkeeping (wavefronts arrived, jobs added up).
constexpr uint32_t kSmallM = 4;
constexpr uint32_t kSmallBufOff = kSlotTableBytes + kSegWaves * kWinBytes;
constexpr uint32_t kSmallFlagsOff = kSmallBufOff + kSegWaves * kSmallM * 32 * 4;
constexpr uint32_t kSegLdsBytes = kSmallFlagsOff + 16;
static_assert(kWinRows * 64 % 1024 == 0 && kSegLdsBytes <= kLdsLimit, "windows exceed the LDS");

// What an item reads before its window is known (requested two items ahead, looked at one item ahead).
struct SegRaw {
    uint32_t state, row, row_end;  // per lane, as stored: decoder state, row of the next unread byte at the
                                   // item's first row and at its end
    uint32_t off, depth;           // the tile's body: byte offset in the stream, rows
};
// An item ready to be staged: lane state, window, and whether the hand-scheduled loop can take it.
struct SegItem {
    uint32_t vk, tn;
    uint32_t state;
    int32_t row;
    uint32_t lo, rows;  // first body row of the window, rows in it
    uint64_t base;      // byte offset of the tile body
    bool fast;
};

__device__ __forceinline__ void seg_request(const LinearArgs &a, uint32_t vk, uint32_t tn, int lane, SegRaw &m) {
    const uint32_t tk = vk / a.segs, seg = vk % a.segs, tile = tk * a.tiles_n + tn;
    m.off = a.tile_offsets[tile];
    m.depth = a.tile_max_lens[tile];
    const uint2 *ck = a.ckpt + ((size_t)tile * (a.segs - 1)) * 64 + lane;  // (only read when segs > 1)
    if (seg == 0) {
        m.state = a.states[(size_t)tile * 64 + lane];
        m.row = 0x7fffffffu;
    } else {
        const uint2 v = ck[(size_t)(seg - 1) * 64];
        m.state = v.x;
        m.row = v.y;
    }
    m.row_end = seg + 1 < a.segs ? ck[(size_t)seg * 64].y : 0xffffffffu;
}

// Decode steps this lane's stream has in item vk of column tile tn: the segment's length, less at the ragged
// end of K, none in a column past N.
__device__ __forceinline__ uint32_t seg_steps(const LinearArgs &a, uint32_t vk, uint32_t tn, int lane) {
    const uint32_t tk = vk / a.segs, seg = vk % a.segs;
    const uint32_t half = a.th / 2, seglen = half / a.segs, hsel = lane / 32, c = lane % 32;
    const uint32_t k0 = tk * a.th + hsel * half + seg * seglen;
    return tn * 32 + c < a.N && k0 < a.K ? min(seglen, a.K - k0) : 0u;
}

__device__ __forceinline__ void seg_resolve(const LinearArgs &a, uint32_t vk, uint32_t tn, int lane, const SegRaw &m,
                                            SegItem &it) {
    const uint32_t seglen = a.th / 2 / a.segs;
    it.vk = vk;
    it.tn = tn;
    it.base = m.off;
    uint32_t depth = m.depth;
    if (it.base + (uint64_t)depth * 64 > a.stream_len) depth = 0;  // a body that would run past the stream is not read
    it.state = m.state;
    it.row = min((int32_t)m.row, (int32_t)depth - 1);
    const int32_t row_end = min((int32_t)m.row_end, it.row);
    const bool full = __builtin_amdgcn_ballot_w64(seg_steps(a, vk, tn, lane) != seglen) == 0;
    // rows of the body the item can touch: from the lowest row a lane has reached by the item's end (the byte
    // there is fetched ahead, never used) to the highest row a lane starts at
    const int32_t lo = max(wave_min_i32(row_end), 0), hi = wave_max_i32(it.row);
    it.lo = (uint32_t)lo;
    it.rows = hi >= lo ? (uint32_t)(hi - lo + 1) : 0u;
    it.fast = full && a.fast_ok && it.rows <= kWinRows && seglen % 16 == 0;
}

// Touches the cache lines the item's start will read: its window of the body (lanes 0..55, a 128-byte line
// each) and the first 128 rows of both halves of its sign|mantissa rows (all lanes).  The values are not
// used; the loads bring the lines next to the CU while the previous item still decodes.  Plain global loads
// (a volatile access would become a flat, system-scope load, which the LDS counter of every decode step
// would wait for): the caller keeps the two values alive until the item's loop has run.
__device__ __forceinline__ void seg_touch(const LinearArgs &a, const SegItem &it, int lane, uint32_t &t, uint32_t &t2) {
    t = t2 = 0;
    if (!it.fast) return;
    const uint32_t tk = it.vk / a.segs, seg = it.vk % a.segs, tile = tk * a.tiles_n + it.tn;
    const uint32_t half = a.th / 2, seglen = half / a.segs;
    if ((uint32_t)lane * 128 < it.rows * 64)
        t = *reinterpret_cast<const uint32_t *>(a.stream + it.base + (size_t)it.lo * 64 + lane * 128);
    const uint32_t hsel = lane / 32, line = lane % 32;  // 4 sign|mantissa rows of a tile make a line
    if (line * 4 < seglen)
        t2 = *reinterpret_cast<const uint32_t *>(a.man_tiled + (size_t)tile * a.th * 32 +
                                                 (size_t)(hsel * half + seg * seglen + line * 4) * 32);
}

// The item's window, memory -> LDS as it lies (stage_window).
__device__ __forceinline__ void seg_stage(const LinearArgs &a, const SegItem &it, uint8_t *stage, int lane) {
    stage_window(stage, a.stream + it.base + (size_t)it.lo * 64, it.rows, lane);
}

// One staged item through the hand-scheduled loop, accumulating into acc (and acc2 for x rows 32..63).
template <int MB>
__device__ __forceinline__ void seg_run(const LinearArgs &a, const SegItem &it, const uint8_t *stage, int lane,
                                        f32x16 &acc, f32x16 &acc2) {
    const uint32_t tk = it.vk / a.segs, seg = it.vk % a.segs, tile = tk * a.tiles_n + it.tn;
    const uint32_t half = a.th / 2, seglen = half / a.segs, hsel = lane / 32, c = lane % 32;
    const uint32_t k0 = tk * a.th + hsel * half + seg * seglen;
    FastLane st;
    st.X = it.state << 3;
    const int32_t rel = max(it.row - (int32_t)it.lo, -1);  // this lane's next byte, in rows of the window (-1: none left)
    st.q = (uint32_t)(uintptr_t)stage + (uint32_t)(rel * 64 + lane);
    st.n1 = rel >= 0 ? stage[rel * 64 + lane] : 0;
    const uint32_t m = c;  // row of x this lane feeds to the (first) MFMA
    const bool m_ok = m < a.M, m2_ok = MB == 2 && m + 32 < a.M;
    const uint64_t mbase = reinterpret_cast<uint64_t>(a.man_tiled + (size_t)tile * a.th * 32);
    // readfirstlane returns a signed int: widen through uint32_t, not by sign extension
    const uint32_t mb_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(mbase >> 32));
    const uint32_t mb_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)mbase);
    const uint64_t mb_u = ((uint64_t)mb_hi << 32) | (uint64_t)mb_lo;
    const uint32_t moff = (hsel * half + seg * seglen) * 32 + (c & ~3u);
    const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
    uint64_t xb = reinterpret_cast<uint64_t>(a.x);
    uint32_t xo = ((m_ok ? m : 0) * a.x_stride + k0) * 2u, xo2 = ((m2_ok ? m + 32 : 0) * a.x_stride + k0) * 2u, xstep = 16;
    if (a.xf) {
        const uint32_t kbs = a.K / 8;
        xb = reinterpret_cast<uint64_t>(a.xf);
        xo = ((k0 / 8) * 32 + c) * 16;
        xo2 = xo + kbs * 32 * 16;
        xstep = 32 * 16;
    }
    if (MB == 2)
        linear_tile_asm2(st, acc, acc2, mb_u, moff, xb, xo, xo2, xstep, man_sel, seglen / 8, 64);
    else
        linear_tile_asm(st, acc, mb_u, moff, xb, xo, xstep, man_sel, seglen / 8, 64);
}

// An item that the loop above cannot take (ragged edges, a window larger than kWinRows, a plain-weight run).
template <int MB>
__device__ __forceinline__ void seg_cold_item(const LinearArgs &a, uint32_t vk, uint32_t tn, const uint2 *tab,
                                                        uint8_t *stage, int lane, f32x16 &acc, f32x16 &acc2) {
    linear_one_item<MB, 0, true>(a, vk, tn, tab, stage, lane, acc, acc2);
}

// Jobs.  With VK = tiles_k * segs items per column tile:
//   VK >= 16: a job is one column tile and one chunk of its items, vk in [chunk * 16 R, (chunk + 1) * 16 R);
//     wavefront w takes item chunk * 16 R + 16 r + w in its round r and keeps one accumulator over its R items;
//   VK < 16: a job is 16 / VK neighbouring column tiles with all their items, wavefront w item w % VK of
//     column tile w / VK (R = 1, one chunk).
// At the end of a job the accumulators that belong to one column tile are added through LDS in wavefront
// order and the sum goes to the output (one chunk per column tile) or to plane `chunk` of the fp32
// workspace.  Which wavefront adds what is fixed by the shape and the CU count alone, so the same job on
// a plain bf16 weight (LinearArgs::dense_w) gives the same bits.
struct SegJobs {
    uint32_t VK, R, chunk_items, chunks, cols, per_col, jobs;
    __device__ __forceinline__ void init(const LinearArgs &a) {
        VK = a.tiles_k * a.segs;
        if (VK >= (uint32_t)kSegWaves) {
            R = a.rounds;
            chunk_items = kSegWaves * R;
            chunks = (VK + chunk_items - 1) / chunk_items;  // == a.P
            cols = 1;
            per_col = kSegWaves;
            jobs = a.tiles_n * chunks;
        } else {
            R = 1;
            chunk_items = VK;
            chunks = 1;
            cols = kSegWaves / VK;
            per_col = VK;
            jobs = (a.tiles_n + cols - 1) / cols;
        }
    }
    // item of wavefront `wave` in round r of job `job`: false if there is none
    __device__ __forceinline__ bool item(const LinearArgs &a, uint32_t job, uint32_t r, uint32_t wave, uint32_t &vk,
                                         uint32_t &tn) const {
        if (cols == 1) {
            tn = job % a.tiles_n;
            vk = (job / a.tiles_n) * chunk_items + r * kSegWaves + wave;
            return vk < VK;
        }
        tn = job * cols + wave / per_col;
        vk = wave % per_col;
        return wave < cols * per_col && tn < a.tiles_n;
    }
};

// grid: any number of workgroups (one per CU); workgroup j takes jobs j, j + gridDim.x, ...
// kCold = false: the instance for weights whose every item is known to take the hand-scheduled loop (full
// tiles, windows of at most kWinRows rows: LinearArgs::all_fast).  It holds no code for the guarded path,
// whose registers would otherwise be spilled around every item; an item that does not qualify after all
// (a descriptor that promised too much) is left out rather than staged beyond its window area.
template <int MB, bool kCold>
__global__ __launch_bounds__(kSegWaves *kWave) void fused_linear32_seg_kernel(LinearArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    // (the wavefront's index through readfirstlane: everything derived from it -- jobs, items, tiles -- is then
    // uniform for the compiler too and lives in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave)), lane = threadIdx.x % kWave;
    // the slot table is asked for before anything else: the job arithmetic below runs while it travels
    const bool copy_table = (!kCold || a.dense_w == nullptr) && a.slot_table;
    u32x4 tab0 = {0, 0, 0, 0}, tab1 = {0, 0, 0, 0};
    if (copy_table) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.slot_table);
        tab0 = src[threadIdx.x * 2];
        tab1 = src[threadIdx.x * 2 + 1];
    }
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kWinBytes;
    SegJobs jb;
    jb.init(a);
    const uint32_t my_jobs = blockIdx.x < jb.jobs ? (jb.jobs - blockIdx.x + gridDim.x - 1) / gridDim.x : 0u;
    const uint32_t slots = my_jobs * jb.R;  // this wavefront's sequence of (job, round) slots, some without an item
    auto slot_item = [&](uint32_t sl, uint32_t &vk, uint32_t &tn) {
        return jb.item(a, blockIdx.x + (sl / jb.R) * gridDim.x, sl % jb.R, (uint32_t)wave, vk, tn);
    };
    auto next_slot = [&](uint32_t sl, uint32_t &vk, uint32_t &tn) {  // first slot >= sl that has an item, or `slots`
        while (sl < slots && !slot_item(sl, vk, tn)) ++sl;
        return sl;
    };
    const bool coded = !kCold || a.dense_w == nullptr;

    // the first item's inputs are on their way while the table is copied
    SegRaw raw;
    SegItem nxt;
    nxt.fast = false;
    uint32_t vk_n = 0, tn_n = 0, vk_nn = 0, tn_nn = 0;
    uint32_t s_nxt = next_slot(0, vk_n, tn_n), s_nn = slots;  // the next slot with an item, and the one after
    if (coded && s_nxt < slots) seg_request(a, vk_n, tn_n, lane, raw);
    if (copy_table) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds);
        dst[threadIdx.x * 2] = tab0;
        dst[threadIdx.x * 2 + 1] = tab1;
    } else if (coded) {
        build_slot_table_x8(reinterpret_cast<uint2 *>(lds), a.tables, a.slot_map, threadIdx.x, kSegWaves * kWave);
    }
    if (coded && s_nxt < slots) {
        seg_resolve(a, vk_n, tn_n, lane, raw, nxt);
        s_nn = next_slot(s_nxt + 1, vk_nn, tn_nn);
        if (s_nn < slots) seg_request(a, vk_nn, tn_nn, lane, raw);
    }
    if (threadIdx.x == 0) {
        uint32_t *flags = reinterpret_cast<uint32_t *>(lds + kSmallFlagsOff);
        flags[0] = flags[1] = 0;
    }
    __syncthreads();

    const uint32_t hsel = lane / 32, c = lane % 32;
    f32x16 acc, acc2;
    for (uint32_t sl = 0; sl < slots; ++sl) {
        if (sl % jb.R == 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = acc2[v] = 0.f;
        }
        const uint32_t job = blockIdx.x + (sl / jb.R) * gridDim.x;
        uint32_t vk, tn;
        if (slot_item(sl, vk, tn)) {
            if (kCold && !coded) {
                seg_cold_item<MB>(a, vk, tn, tab, stage, lane, acc, acc2);
            } else {
                // (sl == s_nxt: the slots with an item are visited in order)
                const SegItem cur = nxt;
                if (cur.fast) seg_stage(a, cur, stage, lane);
                uint32_t touched = 0, touched2 = 0;  // (kept apart: adding them would wait for both loads)
                s_nxt = s_nn;
                vk_n = vk_nn;
                tn_n = tn_nn;
                if (s_nxt < slots) {
                    seg_resolve(a, vk_n, tn_n, lane, raw, nxt);
                    seg_touch(a, nxt, lane, touched, touched2);
                    s_nn = next_slot(s_nxt + 1, vk_nn, tn_nn);
                    if (s_nn < slots) seg_request(a, vk_nn, tn_nn, lane, raw);
                }
                if (cur.fast)
                    seg_run<MB>(a, cur, stage, lane, acc, acc2);  // (a wavefront's LDS operations complete in order)
                else if (kCold)
                    seg_cold_item<MB>(a, vk, tn, tab, stage, lane, acc, acc2);
                asm volatile("" ::"v"(touched), "v"(touched2));  // the touching loads end here
            }
        }
        if (sl % jb.R != jb.R - 1) continue;
        // End of a job: add the accumulators of each column tile in wavefront order.  Every wavefront stores
        // its fragment as [v][lane] floats in its own window area; wavefront w then adds row v = w of the
        // fragments of each column tile of the job, which is column (w/4)*8 + (lane/32)*4 + w%4 of that tile
        // for x row lane%32 (MFMA 32x32 result layout: register v of lane l is row (v/4)*8 + (l/32)*4 + v%4,
        // column l%32).
        const uint32_t chunk = jb.cols == 1 ? job / a.tiles_n : 0u;
        if (MB == 1 && a.M <= kSmallM) {
            // Few rows of x: only the lanes of those rows hold sums, 32 per row and wavefront.  They go to a small
            // area of their own and the last wavefront to arrive adds them up -- in wavefront order, like the
            // general case below -- while the others are already on their next job: no barrier.  The area is
            // handed from job to job by the count of jobs added up.
            float *buf = reinterpret_cast<float *>(lds + kSmallBufOff);
            uint32_t *flags = reinterpret_cast<uint32_t *>(lds + kSmallFlagsOff);
            const uint32_t jn = sl / jb.R;  // which of this workgroup's jobs
            // (the wavefront adding up the job before this one is not waiting for us; the wait is bounded all the same.
            // The limit is tested before the flag, so that a limit of 0 gives up whatever the flag says: the forced
            // give-up of the tests does not depend on who got where first)
            for (uint32_t looks = 0;; ++looks) {
                if (looks >= a.wait_limit) {
                    if (lane == 0) atomicOr(&g_device_status, (uint32_t)CI_STATUS_WAIT_GAVE_UP);
                    break;
                }
                if (__hip_atomic_load(&flags[1], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) == jn) break;
                __builtin_amdgcn_s_sleep(2);
            }
            if (c < a.M) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    buf[((uint32_t)wave * kSmallM + c) * 32 + (v / 4) * 8 + hsel * 4 + (v % 4)] = acc[v];
            }
            uint32_t arrived = 0;
            if (lane == 0) arrived = __hip_atomic_fetch_add(&flags[0], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
            arrived = (uint32_t)__builtin_amdgcn_readfirstlane((int)arrived);
            if (arrived == (uint32_t)kSegWaves - 1) {
                const uint32_t per_tile = 32 * a.M;
                for (uint32_t o = lane; o < jb.cols * per_tile; o += kWave) {
                    const uint32_t t = o / per_tile, mg = (o % per_tile) / 32, n32 = o % 32;
                    const uint32_t col_tile = jb.cols == 1 ? job % a.tiles_n : job * jb.cols + t;
                    float sum = 0.f;
                    for (uint32_t i = 0; i < jb.per_col; ++i) sum += buf[((t * jb.per_col + i) * kSmallM + mg) * 32 + n32];
                    const uint32_t n = col_tile * 32 + n32;
                    if (col_tile < a.tiles_n && n < a.N) {
                        if (a.P == 1)
                            a.out[(size_t)mg * a.out_stride + n] = finish_bf16(sum, a.bias, n);
                        else
                            a.partial[((size_t)chunk * a.M + mg) * a.N + n] = sum;
                    }
                }
                if (lane == 0) {
                    __hip_atomic_store(&flags[0], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_store(&flags[1], jn + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
            continue;
        }
        float *red = reinterpret_cast<float *>(lds + kSlotTableBytes);
#pragma unroll
        for (int g = 0; g < MB; ++g) {
            const f32x16 &part = g ? acc2 : acc;
            __syncthreads();  // the window areas are free: every wavefront has left its loop
#pragma unroll
            for (int v = 0; v < 16; ++v) red[(size_t)wave * (kWinBytes / 4) + v * kWave + lane] = part[v];
            __syncthreads();
            for (uint32_t t = 0; t < jb.cols; ++t) {
                const uint32_t col_tile = jb.cols == 1 ? job % a.tiles_n : job * jb.cols + t;
                float sum = 0.f;
                for (uint32_t i = 0; i < jb.per_col; ++i)
                    sum += red[(size_t)(t * jb.per_col + i) * (kWinBytes / 4) + wave * kWave + lane];
                const uint32_t n = col_tile * 32 + (wave / 4) * 8 + hsel * 4 + (wave % 4), mg = c + 32 * g;
                if (col_tile < a.tiles_n && mg < a.M && n < a.N) {
                    if (a.P == 1)
                        a.out[(size_t)mg * a.out_stride + n] = finish_bf16(sum, a.bias, n);
                    else
                        a.partial[((size_t)chunk * a.M + mg) * a.N + n] = sum;
                }
            }
        }
        __syncthreads();  // before the next window is written over the fragments
    }
}

// Any tile width, any tiled layout (TileLayout): one thread per stream, eight rows of x per pass.
// Partial sums (one per stream, i.e. per (k-tile[, half])) go to the fp32 workspace.
// grid: (ceil(streams / 256), ceil(M / 8))
template <int kLayout>
__global__ __launch_bounds__(256) void fused_linear_generic_kernel(LinearArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    constexpr bool kOne = kLayout != kBodyTwo;  // one stream per column over the whole tile height
    const uint32_t spt = (kOne ? 1 : 2) * a.tw;
    const uint64_t sid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (sid >= (uint64_t)a.tiles_k * a.tiles_n * spt) return;
    const uint32_t tile = (uint32_t)(sid / spt), q = (uint32_t)(sid % spt);
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t span = kOne ? a.th : a.th / 2, hsel = kOne ? 0 : q / a.tw, c = q % a.tw;
    const uint32_t col = tn * a.tw + c, k0 = tk * a.th + hsel * span;
    if (col >= a.N) return;
    const uint32_t my_steps = k0 < a.K ? min(span, a.K - k0) : 0;
    const uint32_t m0 = blockIdx.y * 8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t x = a.states[sid];
    const uint8_t *man = a.man_tiled + (size_t)tile * a.th * a.tw + (size_t)hsel * span * a.tw + c;

    auto run = [&](auto &src) {
        for (uint32_t i = 0; i < my_steps; ++i) {
            const uint32_t sym = decode_symbol(x, tab) >> 24;
            src.renorm(x);
            src.renorm(x);
            const float w = bf16_to_f32((uint16_t)assemble_bf16(sym, man[(size_t)i * a.tw]));
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (m0 + j < a.M) acc[j] += bf16_to_f32(a.x[(size_t)(m0 + j) * a.x_stride + k0 + i]) * w;
        }
    };
    if (kLayout == kExactBytes) {
        const uint64_t off = a.stream_offsets[sid];
        uint32_t size = a.stream_sizes[sid];
        if (off + size > a.stream_len) size = 0;
        DenseBytes src;
        src.init(a.stream + off, size);
        run(src);
    } else {
        uint64_t base = a.tile_offsets[tile];
        uint32_t depth = a.tile_max_lens[tile];
        if (base + (uint64_t)depth * spt > a.stream_len) depth = 0;
        GlobalBytes src;
        src.init(a.stream + base, depth, spt, q);
        run(src);
    }
    const uint32_t p = kOne ? tk : tk * 2 + hsel;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        if (m0 + j < a.M) a.partial[((size_t)p * a.M + m0 + j) * a.N + col] = acc[j];
}

// Clears the workspace.  A kernel rather than hipMemsetAsync so that the launch sequence can be
// captured into a HIP graph.
__global__ __launch_bounds__(256) void zero_f32_kernel(float *p, uint64_t n) {
    const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n) p[e] = 0.f;
}

// out[m][n] = bf16(sum_p partial[p][m][n]) (+ bias), p in index order.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *partial, uint32_t P, uint32_t M,
                                                            uint32_t N, const uint16_t *bias, uint16_t *out,
                                                            uint32_t out_stride) {
    const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (uint64_t)M * N) return;
    const uint32_t m = (uint32_t)(e / N), n = (uint32_t)(e % N);
    const size_t plane = (size_t)M * N;
    float s = 0.f;
    uint32_t p = 0;
    // sixteen, then four loads in flight at a time (the sum keeps its order): one load per iteration would
    // make the kernel a chain of P memory latencies
    for (; p + 16 <= P; p += 16) {
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = partial[(size_t)(p + j) * plane + e];
#pragma unroll
        for (int j = 0; j < 16; ++j) s += v[j];
    }
    for (; p + 4 <= P; p += 4) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = partial[(size_t)(p + j) * plane + e];
#pragma unroll
        for (int j = 0; j < 4; ++j) s += v[j];
    }
    for (; p < P; ++p) s += partial[(size_t)p * plane + e];
    out[(size_t)m * out_stride + n] = finish_bf16(s, bias, n);
}

// The same sums, four neighbouring outputs per thread (16-byte loads): for large outputs, where the kernel
// is a stream of P planes and request count matters.  N % 4 == 0, partial 16-byte aligned.  Every output
// is still summed in index order, so both kernels give the same bits.
__global__ __launch_bounds__(64) void splitk_reduce4_kernel(const float *partial, uint32_t P, uint32_t M, uint32_t N,
                                                            const uint16_t *bias, uint16_t *out, uint32_t out_stride) {
    const uint64_t e = ((uint64_t)blockIdx.x * 64 + threadIdx.x) * 4;
    if (e >= (uint64_t)M * N) return;
    const uint32_t m = (uint32_t)(e / N), n = (uint32_t)(e % N);
    const size_t plane = (size_t)M * N;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    uint32_t p = 0;
    for (; p + 8 <= P; p += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const float4 *>(partial + (size_t)(p + j) * plane + e);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s[0] += v[j].x;
            s[1] += v[j].y;
            s[2] += v[j].z;
            s[3] += v[j].w;
        }
    }
    for (; p < P; ++p) {
        const float4 v = *reinterpret_cast<const float4 *>(partial + (size_t)p * plane + e);
        s[0] += v.x;
        s[1] += v.y;
        s[2] += v.z;
        s[3] += v.w;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) out[(size_t)m * out_stride + n + j] = finish_bf16(s[j], bias, n + j);
}

// Same reduction over a bf16 workspace [P][M][N], the layout the reference's own kernels leave
// behind (comp_inference/linear_triton.py:257-264, :303-314).
__global__ __launch_bounds__(256) void splitk_reduce_bf16_kernel(const uint16_t *partial, uint32_t P,
                                                                 uint32_t M, uint32_t N, const uint16_t *bias,
                                                                 uint16_t *out, uint32_t out_stride) {
    const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (uint64_t)M * N) return;
    const uint32_t m = (uint32_t)(e / N), n = (uint32_t)(e % N);
    float s = 0.f;
    for (uint32_t p = 0; p < P; ++p) s += bf16_to_f32(partial[(size_t)p * M * N + e]);
    out[(size_t)m * out_stride + n] = finish_bf16(s, bias, n);
}

// Rows of x from which the fragment copy pays (below, the lanes past M re-read row 0 and one operand
// load touches only M + 1 cache lines), and its size.
constexpr uint32_t kFragMinRows = 17;
// Outputs from which the four-per-thread reduction is used (below, one output per thread keeps more
// wavefronts in flight).
constexpr uint64_t kReduce4MinOutputs = 65536;
static void launch_splitk_reduce(const float *partial, uint32_t P, uint32_t M, uint32_t N, const uint16_t *bias,
                                 uint16_t *out, uint32_t out_stride, hipStream_t s) {
    const uint64_t n = (uint64_t)M * N;
    if (n >= kReduce4MinOutputs && N % 4 == 0 && aligned(partial, 16)) {
        hipLaunchKernelGGL(splitk_reduce4_kernel, dim3((uint32_t)((n / 4 + 63) / 64)), dim3(64), 0, s, partial, P, M, N,
                           bias, out, out_stride);
    } else {
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, partial, P, M, N, bias,
                           out, out_stride);
    }
}

// Groups of 32 rows per pass of fused_linear32_wide_kernel for M rows of x (0: not its case).
static uint32_t wide_groups(uint32_t M) { return M <= 64 ? 0u : M <= 128 ? 4u : 8u; }

// Groups of 32 rows in the fragment copy (the groups past the last row of x are zero): whole passes of the kernel
// that will read it -- four or eight groups where the one-pass kernel may run (`whole_passes`), else the pairs of
// groups that fused_linear32_kernel<2> reads per 64 rows, or the single group of up to 32 rows.
static uint32_t x_fragment_groups(uint32_t M, bool whole_passes) {
    const uint32_t groups = ceil_div(M, 32u), per_pass = whole_passes ? wide_groups(M) : 0u;
    if (per_pass) return ceil_div(groups, per_pass) * per_pass;
    return M > 32 ? 2 * ceil_div(M, 64u) : 1u;
}

// whole_passes = true gives the larger figure: what the size queries answer, whichever kernel then runs.
static size_t x_fragment_bytes(uint32_t M, uint32_t K, bool fast_plan, bool whole_passes = true) {
    if (!fast_plan || M < kFragMinRows || K % 8) return 0;
    return (size_t)x_fragment_groups(M, whole_passes) * 32 * K * 2;
}

struct LinearPlan {
    bool fast, resident, seg16;
    uint32_t kw, nw, P, segs;
    uint32_t rounds;  // seg16: items of a job per wavefront
};

// Rows (decode steps) of the longest item the sixteen-wavefront kernel is given: bf16 weight exponents take
// about 0.35 bytes per symbol, and the lanes of a tile drift apart by some twenty rows, so 256 rows stay
// below kWinRows.  (An item whose window turns out larger takes the guarded path.)
constexpr uint32_t kSegMaxRows = 256;

// fused_linear32_seg_kernel: items per wavefront and job (R) for a weight of VK = tiles_k * segs items per
// column tile on `cus` CUs, by the time the jobs take (rounds of jobs on the chip x R item lengths, and
// about half an item for the reduction launch when a column tile is cut into several chunks); the largest
// R among equals, which leaves the fewest chunks.
static uint32_t seg_rounds(uint32_t VK, uint32_t tiles_n, uint32_t cus) {
    const uint32_t r_max = ceil_div(VK, (uint32_t)kSegWaves);
    uint32_t best = 1;
    uint64_t best_cost = ~0ull;
    for (uint32_t R = 1; R <= r_max; ++R) {
        const uint32_t chunks = ceil_div(VK, kSegWaves * R);
        const uint64_t jobs = (uint64_t)tiles_n * chunks;
        const uint64_t cost = 2 * ((jobs + cus - 1) / cus) * R + (chunks > 1 ? 1 : 0);
        if (cost <= best_cost) {
            best_cost = cost;
            best = R;
        }
    }
    return best;
}

// Tiles from which every tile gets its own wavefront of a resident workgroup: more than a chip of
// 8-wavefront workgroups holds at once (256 CUs x 8).
constexpr uint32_t kResidentMinTiles = 2049;

// segments: 1, or the number of segments the caller's checkpoints cut every stream into.
// cus: CUs of the device, or 0 for the plan that needs the largest workspace.
static LinearPlan plan_linear(uint32_t M, uint32_t K, uint32_t th, uint32_t tw, uint32_t tiles_n, bool dense,
                              bool stream_aligned, uint32_t segments = 1, uint32_t cus = 0) {
    LinearPlan p;
    const uint32_t tiles_k = ceil_div(K, th);
    p.fast = !dense && tw == 32 && th % 16 == 0 && stream_aligned;
    p.segs = 1;
    p.rounds = 1;
    if (p.fast && M <= 64 && segments > 1 && (th / 2) % (16 * segments) == 0) p.segs = segments;
    // items short enough for their windows of the body to fit 7 KB of LDS go to the sixteen-wavefront kernel
    p.seg16 = p.fast && M <= 64 && (th / 2) % (16 * p.segs) == 0 && th / 2 / p.segs <= kSegMaxRows;
    p.resident = !p.seg16 && p.fast && M <= 64 &&
                 (p.segs > 1 || (tiles_k >= 2 && (uint64_t)tiles_k * tiles_n >= kResidentMinTiles));
    if (p.seg16) {
        p.kw = p.nw = 1;
        p.rounds = cus ? seg_rounds(tiles_k * p.segs, tiles_n, cus) : 1;
        p.P = ceil_div(tiles_k * p.segs, kSegWaves * p.rounds);
    } else if (p.resident) {
        p.kw = p.nw = 1;
        p.P = tiles_k * p.segs;
    } else if (p.fast) {
        p.P = ceil_div(tiles_k, kLinMaxWaves);
        p.kw = ceil_div(tiles_k, p.P);
        p.nw = kLinMaxWaves / p.kw;
        if (p.nw > tiles_n) p.nw = tiles_n;
        if (p.nw == 0) p.nw = 1;
    } else {
        p.kw = p.nw = 1;
        p.P = dense ? tiles_k : tiles_k * 2;
    }
    return p;
}

}  // namespace ci

using namespace ci;

extern "C" size_t ci_fused_linear_workspace_bytes_segmented(uint32_t M, uint32_t K, uint32_t N, uint32_t tile_height,
                                                            uint32_t tile_width, int dense, uint32_t segments) {
    if (tile_height == 0 || tile_width == 0) return 0;
    // sized for the slower plan so that the answer does not depend on pointer alignment
    const uint32_t tiles_n = ceil_div(N, tile_width);
    const LinearPlan fast = plan_linear(M, K, tile_height, tile_width, tiles_n, dense != 0, true, segments);
    const LinearPlan slow = plan_linear(M, K, tile_height, tile_width, tiles_n, dense != 0, false, segments);
    const uint32_t P = fast.P > slow.P ? fast.P : slow.P;
    // (the one-thread-per-stream kernel always goes through the workspace, also with a single partial sum:
    // the dense layout with one tile row)
    const size_t partial = (P > 1 || !slow.fast) ? (size_t)P * M * N * sizeof(float) : 0;
    return ((partial + 15) & ~(size_t)15) + x_fragment_bytes(M, K, fast.fast);
}

extern "C" size_t ci_fused_linear_workspace_bytes(uint32_t M, uint32_t K, uint32_t N, uint32_t tile_height,
                                                  uint32_t tile_width, int dense) {
    return ci_fused_linear_workspace_bytes_segmented(M, K, N, tile_height, tile_width, dense, 1);
}

// Segments per stream for a weight of this shape: the fewest (items as long as possible: every item pays
// for its own start) that make an item kSegMaxRows rows or less and the items at least 70 % of the
// wavefronts a chip of 256 CUs x 16 holds; the most that keep an item 64 rows or more if none gets
// there; 1 if the tile shape allows none.
extern "C" uint32_t ci_suggest_segments(uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width) {
    if (tile_height == 0 || tile_width != 32 || tile_height % 16) return 1;
    const uint64_t tiles = (uint64_t)ceil_div(K, tile_height) * ceil_div(N, tile_width);
    const uint32_t half = tile_height / 2;
    uint32_t best = 1;
    for (uint32_t segs = 1; segs <= 64; segs *= 2) {
        if (half % (16 * segs) || half / segs < 64) break;
        if (half / segs > kSegMaxRows) continue;
        best = segs;
        if (tiles * segs * 10 >= 7ull * 256 * kSegWaves) break;
    }
    return best;
}

// Looks of a bounded wait inside a kernel (a look every 128 clocks or so: the default is a fifth of a second, against
// the microsecond a hand-over takes).  ci_debug_wait_limit sets it, for tests that force the give-up path.
static std::atomic<uint32_t> g_wait_limit{1u << 22};

extern "C" uint32_t ci_debug_wait_limit(uint32_t looks) { return g_wait_limit.exchange(looks); }

extern "C" int ci_device_status(uint32_t *h_status, ci_stream_t stream) {
    if (!h_status) return fail(CI_ERR_ARG, "ci_device_status: null result pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    void *word = nullptr;
    CI_HIP(hipGetSymbolAddress(&word, HIP_SYMBOL(g_device_status)));
    CI_HIP(hipMemcpyAsync(h_status, word, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    CI_HIP(hipMemsetAsync(word, 0, sizeof(uint32_t), s));
    CI_HIP(hipStreamSynchronize(s));
    if (*h_status) return fail(CI_ERR_HIP, "a kernel gave up a bounded wait (device status 0x%x): results since the last check are not to be used", *h_status);
    return CI_OK;
}

// Whether more than 64 rows of x go through fused_linear32_wide_kernel (one decode per 128 or 256 rows) instead
// of fused_linear32_kernel<2> once per 64 rows.  Same results bit for bit; off until it has been measured.
static std::atomic<int> g_wide_rows{0};

extern "C" int ci_fused_linear_wide_rows(int enable) { return g_wide_rows.exchange(enable ? 1 : 0); }

static int fused_linear_impl(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                             const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                             const uint32_t *d_tables, const uint8_t *d_slot_map, const uint32_t *d_meta0,
                             const uint32_t *d_meta1, const uint8_t *d_man_tiled, uint32_t th, uint32_t tw,
                             const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                             size_t workspace_bytes, int layout, hipStream_t s, const uint16_t *d_plain_w = nullptr,
                             const void *d_checkpoints = nullptr, uint32_t segments = 1,
                             const void *d_slot_table = nullptr, uint32_t max_window_rows = 0) {
    const bool dense = layout != kBodyTwo;      // one stream per column: one partial per tile row, no 32-column kernels
    const bool exact = layout == kExactBytes;   // d_meta0 / d_meta1 are stream_offsets / stream_sizes
    if (M == 0 || N == 0) return CI_OK;
    if (K == 0) return fail(CI_ERR_ARG, "fused linear: K is 0");
    if (!d_x || !d_out) return fail(CI_ERR_ARG, "fused linear: null pointer");
    if (!d_plain_w) {
        if (!d_states || !d_tables || !d_slot_map || !d_meta0 || !d_meta1 || !d_man_tiled)
            return fail(CI_ERR_ARG, "fused linear: null pointer");
        if (stream_len && !d_stream) return fail(CI_ERR_ARG, "fused linear: null stream");
        if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "fused linear: slot_map must be 4-byte aligned");
    }
    if (th == 0 || tw == 0 || (!dense && (th & 1))) return fail(CI_ERR_ARG, "fused linear: bad tile shape");
    if (x_stride < K || out_stride < N) return fail(CI_ERR_ARG, "fused linear: row stride shorter than the row");

    LinearArgs a;
    a.x = d_x;
    a.M = M;
    a.K = K;
    a.N = N;
    a.x_stride = x_stride;
    a.stream = d_stream;
    a.stream_len = stream_len;
    a.states = d_states;
    a.tables = d_tables;
    a.slot_map = d_slot_map;
    a.tile_offsets = exact ? nullptr : d_meta0;
    a.tile_max_lens = exact ? nullptr : d_meta1;
    a.stream_offsets = exact ? d_meta0 : nullptr;
    a.stream_sizes = exact ? d_meta1 : nullptr;
    a.man_tiled = d_man_tiled;
    a.dense_w = d_plain_w;
    a.bias = d_bias;
    a.out = d_out;
    a.out_stride = out_stride;
    a.th = th;
    a.tw = tw;
    a.tiles_n = ceil_div(N, tw);
    a.tiles_k = ceil_div(K, th);
    a.fast_ok = aligned(d_x, 16) && x_stride % 8 == 0 && aligned(d_man_tiled, 4) &&
                (uint64_t)M * x_stride * 2 < (1ull << 31);
    if (segments == 0) segments = 1;
    if (segments > 1) {
        if (dense || tw != 32 || th % 16 || (th / 2) % (16 * segments))
            return fail(CI_ERR_ARG, "fused linear: %u segments need 32-column tiles whose half height is a multiple of %u",
                        segments, 16 * segments);
        if (!d_plain_w && (!d_checkpoints || !aligned(d_checkpoints, 8)))
            return fail(CI_ERR_ARG, "fused linear: segments without (8-byte aligned) checkpoints");
    }
    // (planned for no device in particular first: the checks below run before the first HIP call)
    LinearPlan p = plan_linear(M, K, th, tw, a.tiles_n, dense, d_plain_w || aligned(d_stream, 16), segments);
    if (d_plain_w && !p.fast)
        return fail(CI_ERR_ARG, "plain-weight linear: only the 32-column tiling (tile height a multiple of 16)");
    a.ckpt = static_cast<const uint2 *>(d_checkpoints);
    a.slot_table = static_cast<const uint2 *>(d_slot_table);
    // no item is ragged (whole tiles in both directions) and none has a window larger than its staging area
    a.all_fast = !d_plain_w && a.fast_ok && K % th == 0 && N % tw == 0 && max_window_rows != 0 &&
                 max_window_rows <= kWinRows;
    a.rounds = p.rounds;
    a.wait_limit = g_wait_limit.load(std::memory_order_relaxed);
    a.segs = p.segs;
    a.kw = p.kw;
    a.nw = p.nw;
    a.P = p.P;
    a.partial = static_cast<float *>(d_workspace);
    // The one-thread-per-stream kernel writes fp32 partial sums and leaves output, bias and rounding to the
    // reduction, also when there is a single partial sum per output.
    bool via_workspace = p.P > 1 || (!p.fast && !p.resident);
    size_t partial_bytes = 0;
    if (via_workspace) {
        partial_bytes = (size_t)p.P * M * N * sizeof(float);
        if (!d_workspace || workspace_bytes < partial_bytes)
            return fail(CI_ERR_CAPACITY, "fused linear: workspace needs %zu bytes, got %zu", partial_bytes, workspace_bytes);
        if (!aligned(d_workspace, 4)) return fail(CI_ERR_ARG, "fused linear: workspace must be 4-byte aligned");
    }
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    if (p.seg16) {  // how a column tile's items are cut into jobs depends on the CUs there are to fill
        p = plan_linear(M, K, th, tw, a.tiles_n, dense, d_plain_w || aligned(d_stream, 16), segments, cus);
        a.P = p.P;
        a.rounds = p.rounds;
        via_workspace = p.P > 1;
        partial_bytes = via_workspace ? (size_t)p.P * M * N * sizeof(float) : 0;
    }
    // the fragment copy of x goes behind the partials when the caller's workspace has room for it
    a.xf = nullptr;
    // (the guarded path reads x in place; whole passes of four or eight groups only where the one-pass kernel is on)
    const bool wide_on = g_wide_rows.load(std::memory_order_relaxed) != 0;
    const size_t frag_bytes = d_plain_w ? 0 : x_fragment_bytes(M, K, p.fast && a.fast_ok, wide_on);
    if (frag_bytes && frag_bytes < (1ull << 31) && d_workspace) {
        uint8_t *at = static_cast<uint8_t *>(d_workspace) + ((partial_bytes + 15) & ~(size_t)15);
        at += (16 - (reinterpret_cast<uintptr_t>(at) & 15)) & 15;
        if (at + frag_bytes <= static_cast<uint8_t *>(d_workspace) + workspace_bytes) {
            const uint32_t total = (uint32_t)(frag_bytes / 16);
            hipLaunchKernelGGL(x_fragments_kernel, dim3(ceil_div(total, 256u)), dim3(256), 0, s, d_x, M, K, x_stride,
                               reinterpret_cast<u32x4 *>(at), total);
            CI_LAUNCH_CHECK("x_fragments_kernel");
            a.xf = reinterpret_cast<const uint16_t *>(at);
        }
    }

    if (p.seg16) {
        const uint32_t VK = a.tiles_k * p.segs;
        const uint32_t jobs = VK >= (uint32_t)kSegWaves ? a.tiles_n * p.P : ceil_div(a.tiles_n, kSegWaves / VK);
        const dim3 grid(jobs < cus ? jobs : cus), block(kSegWaves * kWave);
        const uint32_t lds_bytes = kSegLdsBytes;
#define CI_LAUNCH_SEG(MB_, COLD_)                                                                   \
    do {                                                                                            \
        CI_ALLOW_FULL_LDS((fused_linear32_seg_kernel<MB_, COLD_>));                                 \
        hipLaunchKernelGGL((fused_linear32_seg_kernel<MB_, COLD_>), grid, block, lds_bytes, s, a);  \
    } while (0)
        if (M > 32) {
            if (a.all_fast) CI_LAUNCH_SEG(2, false); else CI_LAUNCH_SEG(2, true);
        } else {
            if (a.all_fast) CI_LAUNCH_SEG(1, false); else CI_LAUNCH_SEG(1, true);
        }
#undef CI_LAUNCH_SEG
        CI_LAUNCH_CHECK("fused_linear32_seg_kernel");
    } else if (p.resident) {
        CI_ALLOW_FULL_LDS(fused_linear32_resident_kernel<1>);
        CI_ALLOW_FULL_LDS(fused_linear32_resident_kernel<2>);
        const dim3 grid(cus), block(kPersistWaves * kWave);
        if (M > 32)
            hipLaunchKernelGGL(fused_linear32_resident_kernel<2>, grid, block, kLdsLimit, s, a);
        else
            hipLaunchKernelGGL(fused_linear32_resident_kernel<1>, grid, block, kLdsLimit, s, a);
        CI_LAUNCH_CHECK("fused_linear32_resident_kernel");
    } else if (p.fast) {
        const uint32_t waves = p.kw * p.nw;
        const uint32_t lds_bytes = kSlotTableBytes + waves * kFastStageBytes;
        CI_ALLOW_FULL_LDS(fused_linear32_kernel<1>);
        CI_ALLOW_FULL_LDS(fused_linear32_kernel<2>);
        CI_ALLOW_FULL_LDS(fused_linear32_wide_kernel<4>);
        CI_ALLOW_FULL_LDS(fused_linear32_wide_kernel<8>);
        const dim3 block(waves * kWave);
        const uint32_t per_pass = wide_groups(M);
        if (per_pass && a.xf && !d_plain_w && wide_on) {
            const dim3 grid(ceil_div(a.tiles_n, p.nw), p.P, ceil_div(M, 32 * per_pass));
            if (per_pass == 4)
                hipLaunchKernelGGL(fused_linear32_wide_kernel<4>, grid, block, lds_bytes, s, a);
            else
                hipLaunchKernelGGL(fused_linear32_wide_kernel<8>, grid, block, lds_bytes, s, a);
            CI_LAUNCH_CHECK("fused_linear32_wide_kernel");
        } else if (M > 32)
            hipLaunchKernelGGL(fused_linear32_kernel<2>, dim3(ceil_div(a.tiles_n, p.nw), p.P, ceil_div(M, 64)), block,
                               lds_bytes, s, a);
        else
            hipLaunchKernelGGL(fused_linear32_kernel<1>, dim3(ceil_div(a.tiles_n, p.nw), p.P, 1), block, lds_bytes, s, a);
        CI_LAUNCH_CHECK("fused_linear32_kernel");
    } else {
        const uint64_t streams = (uint64_t)a.tiles_k * a.tiles_n * (dense ? 1 : 2) * tw;
        const dim3 grid((uint32_t)((streams + 255) / 256), ceil_div(M, 8)), block(256);
        // columns >= N and empty half tiles leave their slots untouched: start from zero
        const uint64_t nz = (uint64_t)p.P * M * N;
        hipLaunchKernelGGL(zero_f32_kernel, dim3((uint32_t)((nz + 255) / 256)), dim3(256), 0, s, a.partial, nz);
        CI_LAUNCH_CHECK("zero_f32_kernel");
        if (layout == kExactBytes)
            hipLaunchKernelGGL(fused_linear_generic_kernel<kExactBytes>, grid, block, 0, s, a);
        else if (layout == kBodyOne)
            hipLaunchKernelGGL(fused_linear_generic_kernel<kBodyOne>, grid, block, 0, s, a);
        else
            hipLaunchKernelGGL(fused_linear_generic_kernel<kBodyTwo>, grid, block, 0, s, a);
        CI_LAUNCH_CHECK("fused_linear_generic_kernel");
    }
    if (via_workspace) {
        launch_splitk_reduce(a.partial, p.P, M, N, d_bias, d_out, out_stride, s);
        CI_LAUNCH_CHECK("splitk_reduce_kernel");
    }
    return CI_OK;
}

extern "C" int ci_fused_linear_ilp2(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                    const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                    const uint32_t *d_tables, const uint8_t *d_slot_map,
                                    const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                    const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                                    const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                    void *d_workspace, size_t workspace_bytes, ci_stream_t stream) {
    return fused_linear_impl(d_x, M, K, N, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                             d_tile_offsets, d_tile_max_lens, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                             out_stride, d_workspace, workspace_bytes, false, static_cast<hipStream_t>(stream));
}

extern "C" int ci_fused_linear_dense(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                     const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                     const uint32_t *d_tables, const uint8_t *d_slot_map,
                                     const uint32_t *d_stream_offsets, const uint32_t *d_stream_sizes,
                                     const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                                     const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                     void *d_workspace, size_t workspace_bytes, ci_stream_t stream) {
    return fused_linear_impl(d_x, M, K, N, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                             d_stream_offsets, d_stream_sizes, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                             out_stride, d_workspace, workspace_bytes, true, static_cast<hipStream_t>(stream));
}

extern "C" int ci_fused_linear_one(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                   const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                   const uint32_t *d_tables, const uint8_t *d_slot_map,
                                   const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                   const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                                   const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                   void *d_workspace, size_t workspace_bytes, ci_stream_t stream) {
    return fused_linear_impl(d_x, M, K, N, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                             d_tile_offsets, d_tile_max_lens, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                             out_stride, d_workspace, workspace_bytes, kBodyOne, static_cast<hipStream_t>(stream));
}

extern "C" int ci_fused_linear_ilp2_segmented(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                              const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                              const uint32_t *d_tables, const uint8_t *d_slot_map,
                                              const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                              const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                                              const void *d_checkpoints, uint32_t segments, const uint16_t *d_bias,
                                              uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                              size_t workspace_bytes, ci_stream_t stream) {
    return fused_linear_impl(d_x, M, K, N, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                             d_tile_offsets, d_tile_max_lens, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                             out_stride, d_workspace, workspace_bytes, false, static_cast<hipStream_t>(stream), nullptr,
                             d_checkpoints, segments);
}

namespace ci {
__global__ __launch_bounds__(256) void slot_table_kernel(const uint32_t *tables, const uint8_t *slot_map, uint2 *out) {
    build_slot_table_x8(out, tables, slot_map, blockIdx.x * 256 + threadIdx.x, gridDim.x * 256);
}
}  // namespace ci

extern "C" int ci_build_slot_table(const uint32_t *d_tables, const uint8_t *d_slot_map, void *d_slot_table,
                                   size_t slot_table_bytes, ci_stream_t stream) {
    if (!d_tables || !d_slot_map || !d_slot_table) return fail(CI_ERR_ARG, "ci_build_slot_table: null pointer");
    if (slot_table_bytes < CI_SLOT_TABLE_BYTES)
        return fail(CI_ERR_CAPACITY, "ci_build_slot_table: the table takes %d bytes, got %zu", CI_SLOT_TABLE_BYTES,
                    slot_table_bytes);
    if (!aligned(d_slot_map, 4) || !aligned(d_slot_table, 16))
        return fail(CI_ERR_ARG, "ci_build_slot_table: slot_map must be 4-byte, the table 16-byte aligned");
    hipLaunchKernelGGL(slot_table_kernel, dim3(4), dim3(256), 0, static_cast<hipStream_t>(stream), d_tables, d_slot_map,
                       static_cast<uint2 *>(d_slot_table));
    CI_LAUNCH_CHECK("slot_table_kernel");
    return CI_OK;
}

namespace ci {
// One wavefront per item (segment of the 64 streams of a tile): the rows of the tile body the item can touch,
// as the sixteen-wavefront kernel works them out before staging; the maximum over all items whose 64 streams
// all run the segment's full length, at least 1.  (An item at a ragged edge of the shape is never staged:
// every kernel gives it to a path that reads the body in place.  Its window would count for nothing and can
// be the whole body: the lanes of a stream without symbols stay where they start.)
__global__ __launch_bounds__(256) void window_rows_kernel(LinearArgs a, uint32_t num_items, uint32_t *out) {
    const uint32_t item = blockIdx.x * 4 + threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    if (item >= num_items) return;  // (whole wavefronts)
    const uint32_t vk = item / a.tiles_n, tn = item % a.tiles_n;
    SegRaw raw;
    seg_request(a, vk, tn, lane, raw);
    SegItem it;
    seg_resolve(a, vk, tn, lane, raw, it);
    const bool full = __builtin_amdgcn_ballot_w64(seg_steps(a, vk, tn, lane) != a.th / 2 / a.segs) == 0;
    if (lane == 0) atomicMax(out, full && it.rows > 1u ? it.rows : 1u);
}
}  // namespace ci

extern "C" int ci_max_window_rows(const ci_tiled_weight *w, uint32_t *d_rows, ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (!d_rows || !aligned(d_rows, 4)) return fail(CI_ERR_ARG, "ci_max_window_rows: null or unaligned result pointer");
    if (w->tile_width != 32) return fail(CI_ERR_ARG, "ci_max_window_rows: 32-column tiles only");
    const uint32_t segs = w->segments > 1 ? w->segments : 1;
    if ((w->tile_height / 2) % segs) return fail(CI_ERR_ARG, "ci_max_window_rows: half a tile does not split into %u segments", segs);
    LinearArgs a{};
    a.K = w->K;
    a.N = w->N;
    a.th = w->tile_height;
    a.tw = w->tile_width;
    a.tiles_n = ceil_div(w->N, w->tile_width);
    a.tiles_k = ceil_div(w->K, w->tile_height);
    a.segs = segs;
    a.stream = w->d_stream;
    a.stream_len = w->stream_len;
    a.states = w->d_states;
    a.tile_offsets = w->d_tile_offsets;
    a.tile_max_lens = w->d_tile_max_lens;
    a.ckpt = static_cast<const uint2 *>(segs > 1 ? w->d_checkpoints : nullptr);
    a.fast_ok = true;
    const uint64_t items = (uint64_t)a.tiles_k * segs * a.tiles_n;
    if (items > 0xffffffffull / 4) return fail(CI_ERR_ARG, "ci_max_window_rows: too many items");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(zero_f32_kernel, dim3(1), dim3(256), 0, s, reinterpret_cast<float *>(d_rows), (uint64_t)1);
    CI_LAUNCH_CHECK("zero_f32_kernel");
    hipLaunchKernelGGL(window_rows_kernel, dim3((uint32_t)((items + 3) / 4)), dim3(256), 0, s, a, (uint32_t)items, d_rows);
    CI_LAUNCH_CHECK("window_rows_kernel");
    return CI_OK;
}

extern "C" int ci_tiled_weight_check(const ci_tiled_weight *w) {
    if (!w) return fail(CI_ERR_ARG, "weight descriptor: null");
    if (w->K == 0 || w->N == 0 || w->tile_height == 0 || w->tile_width == 0 || (w->tile_height & 1))
        return fail(CI_ERR_ARG, "weight descriptor: bad shape %u x %u, tile %u x %u", w->K, w->N, w->tile_height,
                    w->tile_width);
    const uint64_t tiles = (uint64_t)ceil_div(w->K, w->tile_height) * ceil_div(w->N, w->tile_width);
    if (!w->d_states || !w->d_tables || !w->d_slot_map || !w->d_tile_offsets || !w->d_tile_max_lens)
        return fail(CI_ERR_ARG, "weight descriptor: null pointer");
    // (a weight without sign|mantissa plane can only be decoded to its exponent plane)
    if (!w->d_man_tiled && w->man_len) return fail(CI_ERR_ARG, "weight descriptor: null sign|mantissa plane of %llu bytes",
                                                  (unsigned long long)w->man_len);
    if (w->stream_len && !w->d_stream) return fail(CI_ERR_ARG, "weight descriptor: null stream");
    if (!aligned(w->d_slot_map, 4)) return fail(CI_ERR_ARG, "weight descriptor: slot_map must be 4-byte aligned");
    if (w->n_states < tiles * 2 * w->tile_width)
        return fail(CI_ERR_ARG, "weight descriptor: %llu states, the shape has %llu streams",
                    (unsigned long long)w->n_states, (unsigned long long)(tiles * 2 * w->tile_width));
    if (w->n_tiles < tiles)
        return fail(CI_ERR_ARG, "weight descriptor: tile metadata for %llu tiles, the shape has %llu",
                    (unsigned long long)w->n_tiles, (unsigned long long)tiles);
    if (w->d_man_tiled && w->man_len < tiles * w->tile_height * w->tile_width)
        return fail(CI_ERR_ARG, "weight descriptor: sign|mantissa plane of %llu bytes, the tiles take %llu",
                    (unsigned long long)w->man_len, (unsigned long long)(tiles * w->tile_height * w->tile_width));
    if (w->segments > 1) {
        if (!w->d_checkpoints || !aligned(w->d_checkpoints, 8))
            return fail(CI_ERR_ARG, "weight descriptor: segments without (8-byte aligned) checkpoints");
        const size_t need = ci_checkpoint_bytes(w->K, w->N, w->tile_height, w->tile_width, w->segments);
        if (need == 0 || w->checkpoint_bytes != need)
            return fail(CI_ERR_ARG, "weight descriptor: checkpoints of %llu bytes, %u segments of this shape take %zu",
                        (unsigned long long)w->checkpoint_bytes, w->segments, need);
    }
    if (w->d_slot_table && (w->slot_table_bytes != CI_SLOT_TABLE_BYTES || !aligned(w->d_slot_table, 16)))
        return fail(CI_ERR_ARG, "weight descriptor: the slot table is %d bytes, 16-byte aligned", CI_SLOT_TABLE_BYTES);
    return CI_OK;
}

extern "C" int ci_fused_linear_tiled(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M, uint32_t x_stride,
                                     const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                     size_t workspace_bytes, ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (!w->d_man_tiled) return fail(CI_ERR_ARG, "fused linear: the weight has no sign|mantissa plane");
    return fused_linear_impl(d_x, M, w->K, w->N, x_stride, w->d_stream, w->stream_len, w->d_states, w->d_tables,
                             w->d_slot_map, w->d_tile_offsets, w->d_tile_max_lens, w->d_man_tiled, w->tile_height,
                             w->tile_width, d_bias, d_out, out_stride, d_workspace, workspace_bytes, false,
                             static_cast<hipStream_t>(stream), nullptr, w->segments > 1 ? w->d_checkpoints : nullptr,
                             w->segments > 1 ? w->segments : 1, w->d_slot_table, w->max_window_rows);
}

// ---- an entry point that allocates nothing ----------------------------------------------------------
// For callers that cannot allocate device memory (code under graph capture, tight serving loops): the
// fused linear with its workspace -- fp32 partial sums and the fragment copy of x -- in a fixed array of
// device memory that belongs to the library.  Every GPU the library runs on holds its own copy of the
// array at its own address until the process ends; the address is asked for once per device.  Calls on one
// GPU share that GPU's array, so two of them must not overlap in time (different streams, or threads).
static __device__ __align__(256) uint8_t scratch[CI_NOALLOC_SCRATCH_BYTES];

namespace ci {
constexpr int kMaxScratchDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxScratchDevices];

// Device address of `scratch` on the current device.
static int scratch_address(void **out) {
    int dev = 0;
    CI_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxScratchDevices) return fail(CI_ERR_ARG, "no-allocation linear: device index %d", dev);
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        CI_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));  // (two threads asking at once get the same answer)
        if (!ptr) return fail(CI_ERR_HIP, "no-allocation linear: the scratch array has no device address");
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return CI_OK;
}
}  // namespace ci

// The set-up of the entry point below for the current device (the address of the scratch array), outside any graph
// capture: ci_check_device does it too, so a process that has checked its device is ready.
extern "C" int ci_fused_linear_noalloc_init(void) {
    void *ws = nullptr;
    return scratch_address(&ws);
}

extern "C" int ci_fused_linear_tiled_noalloc(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M,
                                             uint32_t x_stride, const uint16_t *d_bias, uint16_t *d_out,
                                             uint32_t out_stride, ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (!w->d_man_tiled) return fail(CI_ERR_ARG, "fused linear: the weight has no sign|mantissa plane");
    const uint32_t segments = w->segments > 1 ? w->segments : 1;
    const size_t need = ci_fused_linear_workspace_bytes_segmented(M, w->K, w->N, w->tile_height, w->tile_width, 0, segments);
    if (need > (size_t)CI_NOALLOC_SCRATCH_BYTES)
        return fail(CI_ERR_CAPACITY,
                    "no-allocation linear: %u rows of x on a %u x %u weight take %zu bytes of workspace, the library's "
                    "fixed scratch array has %zu; use ci_fused_linear_tiled with a workspace of the caller's",
                    M, w->K, w->N, need, (size_t)CI_NOALLOC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (int rc = scratch_address(&ws)) return rc;
    // (every kernel of the plan writes the partial sums it later reads, or clears them first with a kernel of
    // its own: what an earlier call left in the array is never read)
    return fused_linear_impl(d_x, M, w->K, w->N, x_stride, w->d_stream, w->stream_len, w->d_states, w->d_tables,
                             w->d_slot_map, w->d_tile_offsets, w->d_tile_max_lens, w->d_man_tiled, w->tile_height,
                             w->tile_width, d_bias, d_out, out_stride, ws, (size_t)CI_NOALLOC_SCRATCH_BYTES, false,
                             static_cast<hipStream_t>(stream), nullptr, segments > 1 ? w->d_checkpoints : nullptr,
                             segments, w->d_slot_table, w->max_window_rows);
}

extern "C" int ci_plain_linear_same_order(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                          const uint16_t *d_w, uint32_t tile_height, uint32_t tile_width,
                                          uint32_t segments, const uint16_t *d_bias, uint16_t *d_out,
                                          uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                          ci_stream_t stream) {
    if (!d_w) return fail(CI_ERR_ARG, "plain-weight linear: null weight");
    return fused_linear_impl(d_x, M, K, N, x_stride, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                             tile_height, tile_width, d_bias, d_out, out_stride, d_workspace, workspace_bytes, false,
                             static_cast<hipStream_t>(stream), d_w, nullptr, segments);
}

extern "C" int ci_splitk_reduce(const void *d_partial, int partial_is_bf16, uint32_t P, uint32_t M, uint32_t N,
                                const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                ci_stream_t stream) {
    if (M == 0 || N == 0) return CI_OK;
    if (!d_partial || !d_out || P == 0) return fail(CI_ERR_ARG, "ci_splitk_reduce: null pointer or P == 0");
    if (out_stride < N) return fail(CI_ERR_ARG, "ci_splitk_reduce: row stride shorter than the row");
    const uint64_t n = (uint64_t)M * N;
    const dim3 grid((uint32_t)((n + 255) / 256)), block(256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (partial_is_bf16)
        hipLaunchKernelGGL(splitk_reduce_bf16_kernel, grid, block, 0, s, static_cast<const uint16_t *>(d_partial), P,
                           M, N, d_bias, d_out, out_stride);
    else
        launch_splitk_reduce(static_cast<const float *>(d_partial), P, M, N, d_bias, d_out, out_stride, s);
    CI_LAUNCH_CHECK("splitk_reduce_kernel");
    return CI_OK;
}
