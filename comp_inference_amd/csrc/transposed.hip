// Fused decompress + linear against a weight stored row-per-output ("transposed", the layout of
// an embedding table reused as LM head) on gfx950.
//
// out[M, V] = x[M, H] * W^T with W tiled as [V rows, H columns].  Replaces
// fused_rans_linear_transposed_triton / fused_rans_matmul_transposed_kernel_ilp2_splitk
// (comp_inference/transposed_linear_triton.py:187-435) and the dense variant (:660-883).
//
// The reference gives every 64 output rows their own program, which first discards all decode
// steps above its rows.  Here one wavefront walks one tile exactly once: at step i lane (half, c)
// holds W[v_i, c]; the products with x[m, c] are summed over the 32 lanes of the half -- eight rows
// at a time, with a cross-lane reduction that folds the eight sums together -- and written as the
// partial sum of output row v_i for this column tile.
// Partials go to a workspace [tiles_n][M][V] (fp32) and are summed in tile order by the split-K
// reduction kernel, so the result does not depend on scheduling.
#include "ci_common.h"
#include "rans_device.h"
#include "fast_tile.h"

namespace ci {

constexpr int kTrRows = 4;  // rows of x handled per pass

struct TransArgs {
    const uint16_t *x;
    uint32_t M, H, V, x_stride;  // M = rows of this pass (<= kTrRows)
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
    float *partial;  // [P][M][V]
    uint32_t th, tw, tiles_n, tiles_k, num_tiles;
    // Verification aid: when set, the weights are read from this plain bf16 [V, H] matrix instead of
    // being decoded (same products, same reduction); none of the compressed operands is touched.
    const uint16_t *dense_w;
    // Decoder checkpoints (the index of ci_build_checkpoints_ilp2) for the sixteen-wavefront kernel: every
    // stream cut into segs segments of seglen rows; slot_table: the 32 KB table kept beside the weight, or null.
    const uint2 *ckpt;
    uint32_t segs, seglen;
    const uint2 *slot_table;
    uint32_t first_tile;  // trans32_kernel: tiles below this one are not its work
};

template <int kCtrl>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xF, 0xF, false);
    return v + __int_as_float(moved);
}

__device__ __forceinline__ float weight_f32(uint32_t sym, uint32_t man) {
    return __uint_as_float(((man & 0x80u) << 24) | (sym << 23) | ((man & 0x7Fu) << 16));
}

// a + b after exchanging the second 16-lane row of `a` with the first 16-lane row of `b`: lanes of
// the first row of each 32-lane group end up with a[l] + a[l + 16], lanes of the second row with
// b[l - 16] + b[l].
__device__ __forceinline__ float swap16_add(float a, float b) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sums of eight values per lane over the 32 lanes of each half wave, all eight at once: every
// level adds lane pairs and at the same time halves the number of values a lane carries, so the
// whole reduction is 19 instructions instead of 8 x 5.  On return every lane of the quad
// (r, b8, b4) -- r = 16-lane row of the half, b8 = 8-lane group of the row, b4 = quad of the group --
// holds the total of value 4 * b4 + 2 * b8 + r.
__device__ __forceinline__ float reduce8_over32(const float (&p)[8], bool b8, bool b4) {
    const float s0 = swap16_add(p[0], p[1]), s1 = swap16_add(p[2], p[3]);
    const float s2 = swap16_add(p[4], p[5]), s3 = swap16_add(p[6], p[7]);
    // every cross-lane add runs on all lanes; only the choice between two results is per lane
    const float a0 = dpp_add<0x128>(s0), a1 = dpp_add<0x128>(s1);  // row_ror:8
    const float a2 = dpp_add<0x128>(s2), a3 = dpp_add<0x128>(s3);
    const float t0 = b8 ? a1 : a0, t1 = b8 ? a3 : a2;
    const float c0 = dpp_add<0x104>(t0), c1 = dpp_add<0x114>(t1);  // row_shl:4, row_shr:4
    float u = b4 ? c1 : c0;
    u = dpp_add<0x4E>(u);     // quad_perm [2,3,0,1]
    return dpp_add<0xB1>(u);  // quad_perm [1,0,3,2]
}

// Eight rows of one tile (w[d] = this lane's weights of rows 2d, 2d + 1 as two bf16) against MB rows
// of x: products, the eight-at-once reduction, and one store per quad.  `limit` = rows of the block
// that exist (8 in a full tile).
template <int MB>
__device__ __forceinline__ void trans_emit8(const uint32_t (&w)[4], const uint32_t (&xb)[MB], uint32_t M, uint32_t V,
                                            float *dst_blk, uint32_t limit, int lane) {
    const bool b8 = (lane & 8) != 0, b4 = (lane & 4) != 0;
    const uint32_t j = 4u * b4 + 2u * b8 + ((lane >> 4) & 1u);  // which of the 8 rows this quad ends up with
    const bool writer = (lane & 3) == 0 && j < limit;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const float xf = __uint_as_float(xb[m] << 16);
        float p[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) {  // a bf16 x bf16 product is exact in fp32
            p[2 * d] = __uint_as_float(w[d] << 16) * xf;
            p[2 * d + 1] = __uint_as_float(w[d] & 0xFFFF0000u) * xf;
        }
        const float total = reduce8_over32(p, b8, b4);
        if (writer && m < (int)M) dst_blk[(size_t)m * V + j] = total;
    }
}

// The fast path's variant: the same products and reduction, but the eight sums of a block stay in
// registers -- block b of a group of four in lane b of every quad -- and one store per four blocks writes
// 32 consecutive rows from the 32 lanes of a half: whole 128-byte lines instead of 32-byte pieces.
// `keep` carries the sums between the calls of a group; blk = index of the block in the half tile.
template <int MB>
__device__ __forceinline__ void trans_emit8_lines(const uint32_t (&w)[4], const uint32_t (&xb)[MB], uint32_t M, uint32_t V,
                                                  float *dst, uint32_t blk, float (&keep)[MB], int lane) {
    const bool b8 = (lane & 8) != 0, b4 = (lane & 4) != 0;
    const uint32_t j = 4u * b4 + 2u * b8 + ((lane >> 4) & 1u);  // which of the 8 rows this quad ends up with
    const bool mine = (uint32_t)(lane & 3) == (blk & 3u);
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        const float xf = __uint_as_float(xb[m] << 16);
        float p[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) {  // a bf16 x bf16 product is exact in fp32
            p[2 * d] = __uint_as_float(w[d] << 16) * xf;
            p[2 * d + 1] = __uint_as_float(w[d] & 0xFFFF0000u) * xf;
        }
        const float total = reduce8_over32(p, b8, b4);
        keep[m] = mine ? total : keep[m];
        if ((blk & 3u) == 3u && m < (int)M) dst[(size_t)m * V + (blk - 3u) * 8u + 8u * (uint32_t)(lane & 3) + j] = keep[m];
    }
}

// One tile: wave walks it once, eight rows at a time.  Fast path: the eight steps run through the
// hand-scheduled loop; otherwise guarded steps.  Both feed the same products and the same
// reduction, so a tile's partial sums do not depend on the path it took.
template <int MB, uint32_t kStride>
__device__ __forceinline__ void trans_one_tile(const TransArgs &a, uint32_t tile, const uint2 *tab, uint8_t *stage,
                                               int lane) {
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t half = a.th / 2, hsel = lane / 32, c = lane % 32;
    const uint32_t v0 = tk * a.th + hsel * half, h = tn * 32 + c;
    const uint64_t base = a.dense_w ? 0 : a.tile_offsets[tile];
    uint32_t depth = a.dense_w ? 0 : a.tile_max_lens[tile];
    const uint32_t state = a.dense_w ? 0 : a.states[(size_t)tile * 64 + lane];
    if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;
    uint32_t my_steps = 0;
    if (v0 < a.V) my_steps = min(half, a.V - v0);  // rows of this lane's half (same for its 32 lanes)
    const bool full = __builtin_amdgcn_ballot_w64(my_steps != half || h >= a.H) == 0;
    // (half % 32: the fast path stores groups of four eight-row blocks)
    const bool fast = full && depth >= 2 && depth < kStride && half % 32 == 0 && (uint32_t)(uintptr_t)tab == 0 &&
                      !a.dense_w;

    uint32_t xb[MB];  // bf16 bits of x[m, h]
#pragma unroll
    for (int m = 0; m < MB; ++m) xb[m] = (m < (int)a.M && h < a.H) ? a.x[(size_t)m * a.x_stride + h] : 0u;
    const uint8_t *man_tile = a.man_tiled + (size_t)tile * a.th * 32 + (size_t)hsel * half * 32;
    float *dst = a.partial + (size_t)tn * a.M * a.V + v0;  // + m * V + i

    if (fast) {
        stage_body<kStride>(stage, a.stream + base, depth, lane);
        FastLane st;
        st.init<kStride>(stage, depth, lane, state);
        const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
        const uint32_t *mrow = reinterpret_cast<const uint32_t *>(man_tile + (c & ~3u));  // + 8 dwords per row
        const uint32_t nblk = half / 8;
        uint32_t mcur[8], mnext[8];
        float keep[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) keep[m] = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) mcur[r] = mrow[r * 8];
        for (uint32_t blk = 0; blk < nblk; ++blk) {
            // rows of the next block (the last block re-reads its own: stays inside the tile)
            const uint32_t *nrow = mrow + (size_t)(blk + 1 < nblk ? blk + 1 : blk) * 64;
#pragma unroll
            for (int r = 0; r < 8; ++r) mnext[r] = nrow[r * 8];
            uint32_t w[4];
            decode8_weights_asm(st, mcur, man_sel, w);
            trans_emit8_lines<MB>(w, xb, a.M, a.V, dst, blk, keep, lane);
#pragma unroll
            for (int r = 0; r < 8; ++r) mcur[r] = mnext[r];
        }
        return;
    }

    // In the last k-tile the bottom half has fewer rows than the top half: the wave runs to the
    // top half's count, lanes past their own count (or past the last column) contribute zero.
    const uint32_t n_wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)my_steps);
    const bool col_ok = h < a.H;
    const uint8_t *man = man_tile + c;
    const uint16_t *wd = a.dense_w ? a.dense_w + (size_t)v0 * a.H + h : nullptr;  // read below my_steps only
    GlobalBytes src;
    src.init(a.stream + base, depth, 64, lane);
    uint32_t X = state << 3;
    for (uint32_t i0 = 0; i0 < n_wave; i0 += 8) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const uint32_t i = i0 + r;
            uint32_t bits = 0;
            if (col_ok && i < my_steps) {
                if (wd) {
                    bits = wd[(size_t)i * a.H];
                } else {
                    const uint32_t sym = decode_symbol_scaled(X, tab) >> 24;
                    src.renorm_scaled(X);
                    src.renorm_scaled(X);
                    bits = assemble_bf16(sym, man[(size_t)i * 32]);
                }
            }
            w[r / 2] |= bits << (16 * (r & 1));
        }
        trans_emit8<MB>(w, xb, a.M, a.V, dst + i0, my_steps > i0 ? my_steps - i0 : 0u, lane);
    }
}

template <int MB, int kWaves, uint32_t kStride>
__device__ __forceinline__ void trans_wave_tiles(const TransArgs &a, const uint2 *tab, uint8_t *lds, int wave, int lane) {
    if (wave >= kWaves) return;
    uint8_t *stage = persist_stage<kWaves, kStride>(lds, wave);
    for (uint64_t tile = (uint64_t)wave * gridDim.x + blockIdx.x + a.first_tile; tile < a.num_tiles;
         tile += (uint64_t)kWaves * gridDim.x)
        trans_one_tile<MB, kStride>(a, (uint32_t)tile, tab, stage, lane);
}

// grid: at most one workgroup per CU, resident for the whole launch (fast_tile.h); workgroup j
// takes the tiles j, j + gridDim.x, ...
template <int MB>
__global__ __launch_bounds__(kPersistWaves *kWave) void trans32_kernel(TransArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    // (a plain-weight run has no table to build; which wavefront takes which tile does not change a tile's sums)
    const uint32_t cls = a.dense_w ? 0u
                                   : persist_prologue(lds, a.tables, a.slot_map, a.tile_max_lens + a.first_tile,
                                                      a.num_tiles - a.first_tile, blockIdx.x, gridDim.x);
    if (cls == 2u)
        trans_wave_tiles<MB, 8, kDepthDeep>(a, tab, lds, wave, lane);
    else if (cls == 1u)
        trans_wave_tiles<MB, 10, kDepthMedium>(a, tab, lds, wave, lane);
    else
        trans_wave_tiles<MB, 11, kDepthShallow>(a, tab, lds, wave, lane);
}

// ---- sixteen wavefronts per CU, one row of x --------------------------------------------------------------
// The decode step is a chain of dependent instructions and what hides it is the number of wavefronts in flight:
// sixteen leave each 128 VGPRs and, next to the slot table, 7 KB of LDS, which holds the window of the tile body
// that one segment of the 64 streams reads (decoder checkpoints), staged as the rows lie in memory (pointer step
// 64, no transposition).  An item = (tile, segment): seglen rows of both halves.  The caller guarantees, from the
// weight's descriptor, that every item it sends here is whole and has a window of at most kTrWinRows rows; an
// item that does not qualify after all is left out rather than staged beyond its area.  Tiles of a short last
// tile row go to trans32_kernel (first_tile).
constexpr int kTrSegWaves = 16;
constexpr uint32_t kTrWinRows = kPairWinRows;
constexpr uint32_t kTrWinBytes = kTrWinRows * 64;
static_assert(kTrWinBytes % 1024 == 0 && kSlotTableBytes + kTrSegWaves * kTrWinBytes <= kLdsLimit, "windows exceed the LDS");

// kMatrix: the sums across the 32 lanes of a half go through the matrix pipe instead of lane exchanges.  A
// block's weight fragment A[h][k] (k = the block's eight rows of the top half, then of the bottom half) times a
// one-hot B[k][n] is that fragment transposed into the accumulator: after the blocks 2p and 2p + 1,
// D[h][n] = W[row][h] with n < 16 the top half's rows 16 p + n and n >= 16 the bottom half's rows 16 p + n - 16,
// h down the registers (register r of lane l: h = 8 (r / 4) + 4 (l / 32) + r % 4, n = l % 32).  Sixteen
// multiply-adds against the lane's sixteen values of x give half a row sum per lane, the other half sits 32
// lanes away: one v_permlane32_swap and an add over two such pairs of blocks leave 32 consecutive rows of each
// half in the 64 lanes, stored as whole lines.  11 instead of 15 vector instructions per symbol and no chain of
// lane exchanges; the order of the sum over h differs from the other kernels' (not bit-identical to them), and
// 0 x Inf = NaN: a weight with exponent 255 spoils the 31 other rows of its group, so this is for finite weights.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16v __attribute__((ext_vector_type(16)));

template <bool kMatrix>
__device__ __forceinline__ void trans_one_segment(const TransArgs &a, uint32_t tile, uint32_t seg, uint8_t *stage, int lane) {
    const uint32_t tk = tile / a.tiles_n, tn = tile - tk * a.tiles_n;
    const uint32_t half = a.th / 2, seglen = a.seglen, hsel = lane / 32, c = lane % 32;
    const uint32_t v0 = tk * a.th + hsel * half + seg * seglen, h = tn * 32 + c;
    const uint64_t base = a.tile_offsets[tile];
    uint32_t depth = a.tile_max_lens[tile];
    if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;  // a body that would run past the stream is not read
    // decoder state and row of the next unread byte at the segment's first row, and the row reached at its end
    uint32_t state;
    int32_t row = (int32_t)depth - 1, row_end = -1;
    {
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
    const bool whole = __builtin_amdgcn_ballot_w64(v0 >= a.V || a.V - v0 < seglen || h >= a.H) == 0;
    const int32_t lo = max(wave_min_i32(row_end), 0), hi = wave_max_i32(row);
    const uint32_t rows = hi >= lo ? (uint32_t)(hi - lo + 1) : 0u;
    if (!whole || rows > kTrWinRows || seglen % 32 != 0) {
        // Promised not to happen (the host sends whole tile rows of a weight whose largest window is known to fit).
        // A descriptor that promised too much gets zeros for this item's rows -- wrong sums, as documented for an
        // understated window, but never whatever an earlier launch left in the workspace, and nothing staged beyond
        // the window area.
        if (h < a.H && v0 < a.V)
            for (uint32_t i = c; i < min(seglen, a.V - v0); i += 32) a.partial[(size_t)tn * a.V + v0 + i] = 0.f;
        return;
    }
    // the window, memory -> LDS as it lies (rows == 0: a body without bytes, e.g. a constant plane; nothing to stage,
    // and the steps below never ask for a byte)
    stage_window(stage, a.stream + base + (size_t)lo * 64, rows, lane);
    FastLane st;
    const int32_t rel = max(row - lo, -1);  // this lane's next byte, in rows of the window (-1: none left)
    st.X = state << 3;
    st.q = (uint32_t)(uintptr_t)stage + (uint32_t)(rel * 64 + lane);
    st.n1 = rel >= 0 ? stage[rel * 64 + lane] : 0;  // (a wavefront's LDS operations complete in order)

    const uint8_t *man_seg = a.man_tiled + (size_t)tile * a.th * 32 + (size_t)(hsel * half + seg * seglen) * 32;
    const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
    const uint32_t *mrow = reinterpret_cast<const uint32_t *>(man_seg + (c & ~3u));  // + 8 dwords per row
    const uint32_t nblk = seglen / 8;
    uint32_t mcur[8], mnext[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) mcur[r] = mrow[r * 8];
    if constexpr (kMatrix) {
        // this lane's sixteen values of x (the h of its accumulator registers) and its one-hot operands
        float xv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
            xv[r] = __uint_as_float((uint32_t)a.x[tn * 32 + 8 * (r / 4) + 4 * hsel + r % 4] << 16);
        const uint32_t n = c, jstar = n % 8;
        const u32x4 one = {jstar / 2 == 0 ? (jstar & 1 ? 0x3F800000u : 0x3F80u) : 0u,
                           jstar / 2 == 1 ? (jstar & 1 ? 0x3F800000u : 0x3F80u) : 0u,
                           jstar / 2 == 2 ? (jstar & 1 ? 0x3F800000u : 0x3F80u) : 0u,
                           jstar / 2 == 3 ? (jstar & 1 ? 0x3F800000u : 0x3F80u) : 0u};
        const u32x4 none = {0u, 0u, 0u, 0u};
        const bool mine = n / 16 == hsel;  // this lane's column n takes rows of this lane's half k = 8 hsel + j
        const u32x4 hot0 = mine && (n % 16) / 8 == 0 ? one : none, hot1 = mine && (n % 16) / 8 == 1 ? one : none;
        // rows [16 P + L % 16] of half L / 16 (L = lane % 32, P = lane / 32) of every group of 32 rows
        float *dst = a.partial + (size_t)tn * a.V + tk * a.th + (c / 16) * half + seg * seglen + 16 * hsel + c % 16;
        // one block: the next block's sign|mantissa dwords on their way, eight steps, the weights as one operand
        auto block = [&](uint32_t blk) {
            const uint32_t *nrow = mrow + (size_t)(blk + 1 < nblk ? blk + 1 : blk) * 64;
#pragma unroll
            for (int r = 0; r < 8; ++r) mnext[r] = nrow[r * 8];
            uint32_t w[4];
            decode8_weights_asm(st, mcur, man_sel, w, 64);
            // (w[3] is written two instructions before the statement ends: a matrix instruction may read it no sooner
            // than two wait states later, and the compiler does not see inside the statement)
            asm volatile("s_nop 1" : "+v"(w[3]));
#pragma unroll
            for (int r = 0; r < 8; ++r) mcur[r] = mnext[r];
            const u32x4 wv = {w[0], w[1], w[2], w[3]};
            return __builtin_bit_cast(bf16x8_t, wv);
        };
        // two blocks: 16 rows of each half transposed into the accumulator, then this lane's half of their sums
        auto pair_sums = [&](uint32_t blk) {
            const f32x16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            f32x16v acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(block(blk), __builtin_bit_cast(bf16x8_t, hot0), zero, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(block(blk + 1), __builtin_bit_cast(bf16x8_t, hot1), acc, 0, 0, 0);
            float sum = acc[0] * xv[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) sum = __builtin_fmaf(acc[r], xv[r], sum);
            return sum;
        };
        for (uint32_t g = 0; g < nblk / 4; ++g) {  // (seglen is a multiple of 32: whole groups of four blocks)
            const float first = pair_sums(4 * g), second = pair_sums(4 * g + 2);
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(first), __float_as_uint(second), false, false);
            dst[g * 32] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
        }
    } else {
        uint32_t xb[1] = {a.x[h]};  // bf16 bits of x[0, h]
        float *dst = a.partial + (size_t)tn * a.V + v0;  // (M = 1)
        float keep[1] = {0.f};
        for (uint32_t blk = 0; blk < nblk; ++blk) {
            // rows of the next block (the last block re-reads its own: stays inside the segment)
            const uint32_t *nrow = mrow + (size_t)(blk + 1 < nblk ? blk + 1 : blk) * 64;
#pragma unroll
            for (int r = 0; r < 8; ++r) mnext[r] = nrow[r * 8];
            uint32_t w[4];
            decode8_weights_asm(st, mcur, man_sel, w, 64);
            trans_emit8_lines<1>(w, xb, 1, a.V, dst, blk, keep, lane);
#pragma unroll
            for (int r = 0; r < 8; ++r) mcur[r] = mnext[r];
        }
    }
}

// grid: at most one workgroup per CU; workgroup j's wavefront w takes the items w * gridDim + j, + waves * gridDim, ...
// of the tiles below a.first_tile (item = tile * segs + segment).  kMatrix: see trans_one_segment (the accumulator
// and the lane's values of x fit the 128 registers of sixteen wavefronts too).
constexpr int kTrMatWaves = 16;
template <bool kMatrix>
__global__ __launch_bounds__((kMatrix ? kTrMatWaves : kTrSegWaves) * kWave) void trans32_seg_kernel(TransArgs a) {
    constexpr int kWaves = kMatrix ? kTrMatWaves : kTrSegWaves;
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    if (a.slot_table) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.slot_table);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds);
        for (uint32_t e = threadIdx.x; e < kSlotTableBytes / 16; e += kWaves * kWave) dst[e] = src[e];
    } else {
        build_slot_table_x8(reinterpret_cast<uint2 *>(lds), a.tables, a.slot_map, threadIdx.x, kWaves * kWave);
    }
    __syncthreads();
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kTrWinBytes;
    const uint64_t n_items = (uint64_t)a.first_tile * a.segs;
    for (uint64_t item = (uint64_t)wave * gridDim.x + blockIdx.x; item < n_items; item += (uint64_t)kWaves * gridDim.x) {
        const uint32_t tile = (uint32_t)(item / a.segs), seg = (uint32_t)(item - (uint64_t)tile * a.segs);
        trans_one_segment<kMatrix>(a, tile, seg, stage, lane);
    }
}

// Any tile width, any tiled layout (TileLayout): one thread per (tile, half): it decodes the tile's columns
// one after the other and accumulates their products into its own rows of the tile's partial, so
// the summation order is fixed.  Slow; kept for format coverage.
template <int kLayout>
__global__ __launch_bounds__(256) void trans_generic_kernel(TransArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    constexpr bool kOne = kLayout != kBodyTwo;  // one stream per column over the whole tile height
    const uint32_t spt = kOne ? 1u : 2u;
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (uint64_t)a.num_tiles * spt) return;
    const uint32_t tile = (uint32_t)(id / spt), hsel = (uint32_t)(id % spt);
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t span = kOne ? a.th : a.th / 2, v0 = tk * a.th + hsel * span;
    if (v0 >= a.V) return;
    const uint32_t rows = min(span, a.V - v0);
    float *dst = a.partial + (size_t)tn * a.M * a.V + v0;
    for (uint32_t m = 0; m < a.M; ++m)
        for (uint32_t i = 0; i < rows; ++i) dst[(size_t)m * a.V + i] = 0.f;
    for (uint32_t c = 0; c < a.tw; ++c) {  // columns of the tile in order: a fixed summation order
        const uint32_t h = tn * a.tw + c;
        if (h >= a.H) break;
        const uint8_t *man = a.man_tiled + (size_t)tile * a.th * a.tw + (size_t)hsel * span * a.tw + c;
        uint32_t x;
        auto run = [&](auto &src) {
            for (uint32_t i = 0; i < rows; ++i) {
                const uint32_t sym = decode_symbol(x, tab) >> 24;
                src.renorm(x);
                src.renorm(x);
                const float w = weight_f32(sym, man[(size_t)i * a.tw]);
                for (uint32_t m = 0; m < a.M; ++m)
                    dst[(size_t)m * a.V + i] += w * __uint_as_float((uint32_t)a.x[(size_t)m * a.x_stride + h] << 16);
            }
        };
        if (kLayout == kExactBytes) {
            const uint32_t sid = tile * a.tw + c;
            x = a.states[sid];
            const uint64_t off = a.stream_offsets[sid];
            uint32_t size = a.stream_sizes[sid];
            if (off + size > a.stream_len) size = 0;
            DenseBytes src;
            src.init(a.stream + off, size);
            run(src);
        } else {
            const uint32_t row_bytes = spt * a.tw, q = hsel * a.tw + c;
            x = a.states[(size_t)tile * row_bytes + q];
            uint64_t base = a.tile_offsets[tile];
            uint32_t depth = a.tile_max_lens[tile];
            if (base + (uint64_t)depth * row_bytes > a.stream_len) depth = 0;
            GlobalBytes src;
            src.init(a.stream + base, depth, row_bytes, q);
            run(src);
        }
    }
}

}  // namespace ci

using namespace ci;

extern "C" size_t ci_fused_linear_transposed_workspace_bytes(uint32_t M, uint32_t H, uint32_t V,
                                                             uint32_t tile_width) {
    if (tile_width == 0) return 0;
    const uint32_t rows = M < (uint32_t)kTrRows ? M : (uint32_t)kTrRows;
    return (size_t)ceil_div(H, tile_width) * rows * V * sizeof(float);
}

// Whether the sixteen-wavefront kernel for one row of x sums across lanes on the matrix pipe (trans_one_segment).
// Another order of the sum over the hidden dimension (not bit-identical to the other kernels), finite weights only;
// off until it has been measured.
static std::atomic<int> g_matrix_sums{0};

extern "C" int ci_fused_linear_transposed_matrix_sums(int enable) { return g_matrix_sums.exchange(enable ? 1 : 0); }

static int transposed_impl(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V, uint32_t x_stride,
                           const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                           const uint32_t *d_tables, const uint8_t *d_slot_map, const uint32_t *d_meta0,
                           const uint32_t *d_meta1, const uint8_t *d_man_tiled, uint32_t th, uint32_t tw,
                           const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                           size_t workspace_bytes, int layout, ci_stream_t stream,
                           const uint16_t *d_plain_w = nullptr, const void *d_checkpoints = nullptr,
                           uint32_t segments = 1, uint32_t max_window_rows = 0, const void *d_slot_table = nullptr) {
    const bool dense = layout != kBodyTwo;     // one stream per column: one thread per tile in the general kernel
    const bool exact = layout == kExactBytes;  // d_meta0 / d_meta1 are stream_offsets / stream_sizes
    if (M == 0 || V == 0) return CI_OK;
    if (H == 0) return fail(CI_ERR_ARG, "transposed linear: hidden size is 0");
    if (!d_x || !d_out) return fail(CI_ERR_ARG, "transposed linear: null pointer");
    if (!d_plain_w) {
        if (!d_states || !d_tables || !d_slot_map || !d_meta0 || !d_meta1 || !d_man_tiled)
            return fail(CI_ERR_ARG, "transposed linear: null pointer");
        if (stream_len && !d_stream) return fail(CI_ERR_ARG, "transposed linear: null stream");
        if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "transposed linear: slot_map must be 4-byte aligned");
    }
    if (th == 0 || tw == 0 || (!dense && (th & 1))) return fail(CI_ERR_ARG, "transposed linear: bad tile shape");
    if (x_stride < H || out_stride < V) return fail(CI_ERR_ARG, "transposed linear: row stride shorter than the row");
    const size_t need = ci_fused_linear_transposed_workspace_bytes(M, H, V, tw);
    if (!d_workspace || workspace_bytes < need)
        return fail(CI_ERR_CAPACITY, "transposed linear: workspace needs %zu bytes, got %zu", need, workspace_bytes);
    if (!aligned(d_workspace, 4)) return fail(CI_ERR_ARG, "transposed linear: workspace must be 4-byte aligned");

    TransArgs a;
    a.H = H;
    a.V = V;
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
    a.partial = static_cast<float *>(d_workspace);
    a.th = th;
    a.tw = tw;
    a.tiles_n = ceil_div(H, tw);  // column tiles run along the hidden dimension
    a.tiles_k = ceil_div(V, th);
    a.num_tiles = a.tiles_n * a.tiles_k;
    a.ckpt = nullptr;
    a.segs = 1;
    a.seglen = th / 2;
    a.slot_table = static_cast<const uint2 *>(d_slot_table);
    a.first_tile = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool fast = !dense && tw == 32 && (d_plain_w || (aligned(d_stream, 16) && aligned(d_man_tiled, 4)));
    if (d_plain_w && !fast) return fail(CI_ERR_ARG, "plain-weight transposed linear: only the 32-column tiling");
    uint32_t cus = 1;
    if (fast) {
        if (int rc = cu_count(&cus)) return rc;
        CI_ALLOW_FULL_LDS(trans32_kernel<1>);
        CI_ALLOW_FULL_LDS(trans32_kernel<kTrRows>);
    }
    // One row of x on a weight with decoder checkpoints whose largest window is known to fit: the tile rows that
    // are whole go to the sixteen-wavefront kernel, a short last tile row to the kernel below.
    if (fast && M == 1 && !d_plain_w && segments > 1 && d_checkpoints && aligned(d_checkpoints, 8) && th % 2 == 0 &&
        (th / 2) % (32 * segments) == 0 && th / 2 / segments <= 256 && max_window_rows != 0 &&
        max_window_rows <= kTrWinRows && H % 32 == 0 && aligned(d_x, 2)) {
        const uint32_t whole_rows = V / th;  // tile rows without a ragged edge
        if (whole_rows > 0) {
            a.x = d_x;
            a.M = 1;
            a.ckpt = static_cast<const uint2 *>(d_checkpoints);
            a.segs = segments;
            a.seglen = th / 2 / segments;
            a.first_tile = whole_rows * a.tiles_n;
            const uint64_t items = (uint64_t)a.first_tile * segments;
            CI_ALLOW_FULL_LDS(trans32_seg_kernel<false>);
            CI_ALLOW_FULL_LDS(trans32_seg_kernel<true>);
            const dim3 grid((uint32_t)(items < cus ? items : cus));
            if (g_matrix_sums.load(std::memory_order_relaxed))
                hipLaunchKernelGGL(trans32_seg_kernel<true>, grid, dim3(kTrMatWaves * kWave),
                                   kSlotTableBytes + kTrMatWaves * kTrWinBytes, s, a);
            else
                hipLaunchKernelGGL(trans32_seg_kernel<false>, grid, dim3(kTrSegWaves * kWave),
                                   kSlotTableBytes + kTrSegWaves * kTrWinBytes, s, a);
            CI_LAUNCH_CHECK("trans32_seg_kernel");
            a.ckpt = nullptr;
            a.segs = 1;
            a.seglen = th / 2;
        }
    }
    // passes of kTrRows rows of x reuse the workspace one after another on the stream
    for (uint32_t m0 = 0; m0 < M; m0 += kTrRows) {
        a.x = d_x + (size_t)m0 * x_stride;
        a.M = M - m0 < (uint32_t)kTrRows ? M - m0 : (uint32_t)kTrRows;
        if (fast && a.first_tile >= a.num_tiles) {
            // (every tile went to the sixteen-wavefront kernel)
        } else if (fast) {
            const uint32_t left = a.num_tiles - a.first_tile;
            const dim3 grid(left < cus ? left : cus), block(kPersistWaves * kWave);
            if (a.M == 1)
                hipLaunchKernelGGL(trans32_kernel<1>, grid, block, kLdsLimit, s, a);
            else
                hipLaunchKernelGGL(trans32_kernel<kTrRows>, grid, block, kLdsLimit, s, a);
            CI_LAUNCH_CHECK("trans32_kernel");
        } else {
            const uint64_t threads = (uint64_t)a.num_tiles * (dense ? 1 : 2);
            const dim3 grid((uint32_t)((threads + 255) / 256)), block(256);
            if (layout == kExactBytes)
                hipLaunchKernelGGL(trans_generic_kernel<kExactBytes>, grid, block, 0, s, a);
            else if (layout == kBodyOne)
                hipLaunchKernelGGL(trans_generic_kernel<kBodyOne>, grid, block, 0, s, a);
            else
                hipLaunchKernelGGL(trans_generic_kernel<kBodyTwo>, grid, block, 0, s, a);
            CI_LAUNCH_CHECK("trans_generic_kernel");
        }
        int rc = ci_splitk_reduce(a.partial, 0, a.tiles_n, a.M, V, d_bias, d_out + (size_t)m0 * out_stride, out_stride,
                                  stream);
        if (rc) return rc;
    }
    return CI_OK;
}

extern "C" int ci_fused_linear_transposed_ilp2(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                               uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                               const uint32_t *d_states, const uint32_t *d_tables,
                                               const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                               const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled,
                                               uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                               uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                               size_t workspace_bytes, ci_stream_t stream) {
    return transposed_impl(d_x, M, H, V, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                           d_tile_offsets, d_tile_max_lens, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                           out_stride, d_workspace, workspace_bytes, false, stream);
}

extern "C" int ci_fused_linear_transposed_tiled(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M,
                                                uint32_t x_stride, const uint16_t *d_bias, uint16_t *d_out,
                                                uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                                ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (!w->d_man_tiled) return fail(CI_ERR_ARG, "transposed linear: the weight has no sign|mantissa plane");
    // (the weight is stored [V, H]: its rows are the outputs)
    return transposed_impl(d_x, M, w->N, w->K, x_stride, w->d_stream, w->stream_len, w->d_states, w->d_tables,
                           w->d_slot_map, w->d_tile_offsets, w->d_tile_max_lens, w->d_man_tiled, w->tile_height,
                           w->tile_width, d_bias, d_out, out_stride, d_workspace, workspace_bytes, false, stream, nullptr,
                           w->segments > 1 ? w->d_checkpoints : nullptr, w->segments > 1 ? w->segments : 1,
                           w->max_window_rows, w->d_slot_table);
}

extern "C" int ci_fused_linear_transposed_one(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                              uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                              const uint32_t *d_states, const uint32_t *d_tables,
                                              const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                              const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled,
                                              uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                              uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                              size_t workspace_bytes, ci_stream_t stream) {
    return transposed_impl(d_x, M, H, V, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                           d_tile_offsets, d_tile_max_lens, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                           out_stride, d_workspace, workspace_bytes, kBodyOne, stream);
}

extern "C" int ci_fused_linear_transposed_dense(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                                uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                                const uint32_t *d_states, const uint32_t *d_tables,
                                                const uint8_t *d_slot_map, const uint32_t *d_stream_offsets,
                                                const uint32_t *d_stream_sizes, const uint8_t *d_man_tiled,
                                                uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                                uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                                size_t workspace_bytes, ci_stream_t stream) {
    return transposed_impl(d_x, M, H, V, x_stride, d_stream, stream_len, d_states, d_tables, d_slot_map,
                           d_stream_offsets, d_stream_sizes, d_man_tiled, tile_height, tile_width, d_bias, d_out,
                           out_stride, d_workspace, workspace_bytes, true, stream);
}

extern "C" int ci_plain_linear_transposed_same_order(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                                     uint32_t x_stride, const uint16_t *d_w, uint32_t tile_height,
                                                     uint32_t tile_width, const uint16_t *d_bias, uint16_t *d_out,
                                                     uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                                     ci_stream_t stream) {
    if (!d_w) return fail(CI_ERR_ARG, "plain-weight transposed linear: null weight");
    return transposed_impl(d_x, M, H, V, x_stride, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                           tile_height, tile_width, d_bias, d_out, out_stride, d_workspace, workspace_bytes, false,
                           stream, d_w);
}
