// Stand-alone rANS decode of the tiled two-streams-per-column format (gfx950).
//
// Work decomposition for the default 32-column tile: one wavefront per tile.  Lanes 0..31
// own the top-half streams of columns 0..31, lanes 32..63 the bottom-half streams, so one
// stored byte row (64 bytes) is one byte per lane.  One workgroup per CU stays resident for the
// launch and shares one LDS slot table; each wavefront stages a whole tile body in LDS with
// 16-byte coalesced loads, runs the sequential decode out of LDS and takes the next tile.
#include "ci_common.h"
#include "rans_device.h"
#include "fast_tile.h"

namespace ci {

struct DecodeArgs {
    const uint8_t *stream;
    uint64_t stream_len;
    const uint32_t *states;
    const uint32_t *tables;
    const uint8_t *slot_map;
    const uint32_t *tile_offsets;
    const uint32_t *tile_max_lens;
    uint32_t K, N, th, tw, tiles_n, num_tiles;
    uint8_t *out_exp;
    const uint8_t *man_tiled;
    uint16_t *out_bf16;
    uint32_t man_aligned;  // sign|mantissa plane may be read as dwords
    // Decoder checkpoints (see checkpoints_kernel): with segs > 1 every stream is cut into segs segments
    // that are decoded as work items of their own.
    const uint2 *ckpt;
    uint32_t segs;
    uint32_t seglen;  // th / (2 segs): rows of an item (kept here: the kernels would divide for it per item)
};

// Work item of the 32-column kernels: one half (top or bottom rows) of two neighbouring column
// tiles.  Lanes 0..31 own the 32 streams of that half of tile (tk, 2p), lanes 32..63 those of tile
// (tk, 2p + 1), so every decoded row leaves the wavefront as 64 contiguous bytes (128 as bf16).  With
// both halves of ONE tile per wavefront every row is a 32-byte piece of a 128-byte line, and the
// memory side of those partial writes cost a fifth of the kernel's time.
// item = ((tk * pairs + p) * segs + segment) * 2 + half.
//
// With decoder checkpoints an item is one segment of those streams: it starts from the recorded state
// and byte position, stages only the rows of the two bodies its lanes can touch (from the lowest row any
// lane reaches by the segment's end to the highest any lane starts at) and decodes th / (2 segs) rows.
//
// kMerge = false writes the exponent plane; kMerge = true joins it with the tiles' sign|mantissa
// bytes and writes bf16.  Items that do not qualify for the hand-scheduled loop (ragged, odd block
// counts, a window deeper than a lane stride) take the same arithmetic with guarded byte reads from
// global memory.
// ---- sixteen wavefronts per CU ------------------------------------------------------------------------
// The decode step is a chain of dependent instructions, and what hides it is the number of wavefronts a
// CU keeps in flight: sixteen leave each 128 VGPRs and, next to the slot table, 7 KB of LDS.  That holds
// the window of a short item -- a segment of the streams (decoder checkpoints) or the whole streams of a low
// tile -- staged as the rows lie in memory: LDS row r of the window = the item's 32 bytes of row r of body A,
// then those of body B, so lane l finds its bytes at 64 r + l and its pointer moves by 64 per byte.  No
// transposition, no lane exchanges.  kStride == 0 selects this staging in decode_one_item.
constexpr int kDecSegWaves = kPairSegWaves;
constexpr uint32_t kDecWinRows = kPairWinRows;
constexpr uint32_t kDecWinBytes = kPairWinBytes;

template <uint32_t kStride, bool kMerge>
__device__ __forceinline__ void decode_one_item(const DecodeArgs &a, uint32_t item, const uint2 *tab,
                                                uint8_t *stage, int lane) {
    const uint32_t pairs = (a.tiles_n + 1) / 2;
    const uint32_t hsel = item & 1u, seg = (item >> 1) % a.segs, pr = (item >> 1) / a.segs;
    const uint32_t p = pr % pairs, tk = pr / pairs;
    const uint32_t half = a.th / 2, seglen = a.seglen, side = lane / 32, c = lane % 32;
    const uint32_t tn = 2 * p + side, col = tn * 32 + c, row_first = tk * a.th + hsel * half + seg * seglen;
    if (row_first >= a.K) return;  // past the end of a short last tile row
    const bool have_b = 2 * p + 1 < a.tiles_n;
    const uint32_t tile_a = tk * a.tiles_n + 2 * p, tile_b = have_b ? tile_a + 1 : tile_a;
    uint64_t base_a = a.tile_offsets[tile_a], base_b = a.tile_offsets[tile_b];
    uint32_t depth_a = a.tile_max_lens[tile_a], depth_b = a.tile_max_lens[tile_b];
    // A body that would run past the stream is treated as empty rather than read.
    if (base_a + (uint64_t)depth_a * 64 > a.stream_len) depth_a = 0;
    if (base_b + (uint64_t)depth_b * 64 > a.stream_len) depth_b = 0;
    const uint32_t tile = side ? tile_b : tile_a, depth = side ? depth_b : depth_a;
    const uint64_t base = side ? base_b : base_a;
    const uint32_t q = hsel * 32 + c;  // this lane's stream inside its tile
    const bool col_ok = tn < a.tiles_n && col < a.N;
    // decoder state and row of the next unread byte at the segment's first row, and the row the stream
    // has reached at the segment's end
    uint32_t state;
    int32_t row = (int32_t)depth - 1, row_end = -1;
    {
        const uint2 *ck = a.ckpt + ((size_t)tile * (a.segs - 1)) * 64 + q;  // (only read when segs > 1)
        if (seg == 0) {
            state = a.states[(size_t)tile * 64 + q];
        } else {
            const uint2 v = ck[(size_t)(seg - 1) * 64];
            state = v.x;
            row = min((int32_t)v.y, (int32_t)depth - 1);
        }
        if (seg + 1 < a.segs) row_end = min((int32_t)ck[(size_t)seg * 64].y, row);
    }
    const uint32_t steps = min(seglen, a.K - row_first);  // the same for every lane
    // rows of the two bodies this item can touch (one window for both: neighbouring tiles lie alike)
    const int32_t w_lo = max(wave_min_i32(row_end) - 1, 0), w_hi = wave_max_i32(row);
    const uint32_t win_a = (uint32_t)max(min(w_hi + 1, (int32_t)depth_a) - w_lo, 0),
                   win_b = (uint32_t)max(min(w_hi + 1, (int32_t)depth_b) - w_lo, 0);
    constexpr uint32_t kWinLimit = kStride ? kStride : kDecWinRows + 1;  // (rows of a window must stay below it)
    const bool fast = __builtin_amdgcn_ballot_w64(!col_ok) == 0 && steps == seglen && win_a >= 2 && win_b >= 2 &&
                      win_a < kWinLimit && win_b < kWinLimit && seglen % (kMerge ? 8 : 2) == 0 && seglen >= 2 &&
                      (uint64_t)a.K * a.N < (1ull << (kMerge ? 31 : 32)) && (uint32_t)(uintptr_t)tab == 0 &&
                      (!kMerge || a.man_aligned);
    const uint8_t *man_seg =
        kMerge ? a.man_tiled + (size_t)tile * a.th * 32 + (size_t)(hsel * half + seg * seglen) * 32 : nullptr;
    if (fast) {
        const uint32_t deepest = max(win_a, win_b);
        const uint8_t *src_a = a.stream + base_a + (size_t)w_lo * 64, *src_b = a.stream + base_b + (size_t)w_lo * 64;
        FastLane st;
        constexpr uint32_t qdec = kStride ? 1u : 64u;
        if constexpr (kStride != 0) {
            StageRegs body;
            const uint32_t my_depth = (lane & 4) ? win_b : win_a;
#pragma unroll
            for (int grp = 0; grp < stage_groups(kStride); ++grp)
                if ((uint32_t)grp * 128 < deepest) {
                    stage_fetch_pair(body, src_a, win_a, src_b, win_b, hsel, grp * 128, lane);
                    stage_commit<kStride>(body, stage, grp * 128, my_depth, lane);
                }
            // LDS operations of one wavefront complete in order: the reads below see the writes above
            st.init_at<kStride>(stage, row - w_lo + 1, lane, state);
        } else {
            stage_window_pair(stage, src_a, win_a, src_b, win_b, hsel, deepest, lane);
            const int32_t rel = max(row - w_lo, -1);  // this lane's next byte, in rows of the window (-1: none left)
            st.X = state << 3;
            st.q = (uint32_t)(uintptr_t)stage + (uint32_t)(rel * 64 + lane);
            st.n1 = rel >= 0 ? stage[rel * 64 + lane] : 0;
        }
        if (kMerge) {
            // blocks of eight rows: sign|mantissa dwords of the next block are loaded while this one decodes
            const uint32_t man_sel = 0x04040000u + (c & 3u) * 0x01010101u;
            const uint32_t *mrow = reinterpret_cast<const uint32_t *>(man_seg + (c & ~3u));  // + 8 dwords per row
            uint16_t *o = a.out_bf16 + (size_t)row_first * a.N + col;
            const uint32_t nblk = seglen / 8;
            uint32_t mcur[8], mnext[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) mcur[r] = mrow[r * 8];
            for (uint32_t blk = 0; blk < nblk; ++blk) {
                const uint32_t *nrow = mrow + (size_t)(blk + 1 < nblk ? blk + 1 : blk) * 64;
#pragma unroll
                for (int r = 0; r < 8; ++r) mnext[r] = nrow[r * 8];
                uint32_t w[4];
                decode8_weights_asm(st, mcur, man_sel, w, qdec);
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    o[(size_t)(blk * 8 + 2 * d) * a.N] = (uint16_t)w[d];
                    o[(size_t)(blk * 8 + 2 * d + 1) * a.N] = (uint16_t)(w[d] >> 16);
                }
#pragma unroll
                for (int r = 0; r < 8; ++r) mcur[r] = mnext[r];
            }
        } else {
            const uint64_t ob = reinterpret_cast<uint64_t>(a.out_exp + (size_t)row_first * a.N + 2 * p * 32);
            // readfirstlane returns a signed int: widen through uint32_t
            const uint32_t ob_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(ob >> 32));
            const uint32_t ob_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)ob);
            decode_tile_asm(st, ((uint64_t)ob_hi << 32) | (uint64_t)ob_lo, lane, a.N, seglen / 2, qdec);
        }
    } else if (col_ok) {
        GlobalBytes src;
        src.init(a.stream + base, (uint32_t)(row + 1), 64, q);
        uint32_t X = state << 3;
        const size_t o0 = (size_t)row_first * a.N + col;
        for (uint32_t i = 0; i < steps; ++i) {
            const uint32_t sym = decode_symbol_scaled(X, tab) >> 24;
            src.renorm_scaled(X);
            src.renorm_scaled(X);
            if (kMerge)
                a.out_bf16[o0 + (size_t)i * a.N] = (uint16_t)assemble_bf16(sym, man_seg[(size_t)i * 32 + c]);
            else
                a.out_exp[o0 + (size_t)i * a.N] = (uint8_t)sym;
        }
    }
}

__device__ __forceinline__ uint64_t decode_num_pairs(const DecodeArgs &a) {
    return (uint64_t)(a.num_tiles / a.tiles_n) * ((a.tiles_n + 1) / 2);
}

// Workgroup `j` (of the `n_wg` that share this tensor) takes the units j, j + n_wg, ... (a unit = a tile
// pair, or one segment of it); its wavefronts take the workgroup's items in turn (slot = wave,
// wave + kWaves, ...; slot / 2 picks the unit, slot % 2 the half), so the two halves of a unit are staged
// on the same CU at about the same time and the second reader of a body row finds it in that CU's cache.
template <int kWaves, uint32_t kStride, bool kMerge>
__device__ __forceinline__ void decode_wave_tiles(const DecodeArgs &a, uint32_t j, uint32_t n_wg, const uint2 *tab,
                                                  uint8_t *lds, int wave, int lane) {
    if (wave >= kWaves) return;
    uint8_t *stage = persist_stage<kWaves, kStride>(lds, wave);
    const uint64_t n_units = decode_num_pairs(a) * a.segs;  // unit = one segment of a pair, both halves
    for (uint32_t slot = wave;; slot += kWaves) {
        const uint64_t unit = (uint64_t)(slot >> 1) * n_wg + j;
        if (unit >= n_units) break;
        decode_one_item<kStride, kMerge>(a, (uint32_t)unit * 2 + (slot & 1u), tab, stage, lane);
    }
}

// Several tensors in one launch, workgroups resident for the whole launch (fast_tile.h).  A
// stand-alone decode is a chain of tile_height / 2 dependent steps per wavefront whatever the
// tensor's size, so small tensors launched one by one leave most of the chip idle.  Workgroups are
// assigned to tensors by a prefix table in the kernel arguments.
constexpr int kDecBatchMax = 16;
struct DecodeBatchArgs {
    DecodeArgs item[kDecBatchMax];
    uint32_t first_block[kDecBatchMax + 1];
    uint32_t n;
};

template <bool kMerge>
__global__ __launch_bounds__(kPersistWaves *kWave) void decode_tiled32_persist_kernel(DecodeBatchArgs b) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    uint32_t i = 0;
    while (i + 1 < b.n && blockIdx.x >= b.first_block[i + 1]) ++i;
    const DecodeArgs &a = b.item[i];
    const uint32_t j = blockIdx.x - b.first_block[i], n_wg = b.first_block[i + 1] - b.first_block[i];

    uint32_t deepest = 0;
    if (a.segs > 1) {
        // a segment's window is about its share of the body plus the spread between the lanes; an item whose
        // window turns out larger than the class allows takes the guarded path
        for (uint32_t t = tid; t < a.num_tiles; t += kPersistWaves * kWave) deepest = max(deepest, a.tile_max_lens[t]);
        deepest = deepest / a.segs + 40;
    } else {
        const uint32_t pairs = (a.tiles_n + 1) / 2;
        const uint64_t n_pairs = decode_num_pairs(a);
        for (uint64_t pr = (uint64_t)tid * n_wg + j; pr < n_pairs; pr += (uint64_t)kPersistWaves * kWave * n_wg) {
            const uint32_t p = (uint32_t)(pr % pairs), tk = (uint32_t)(pr / pairs);
            const uint32_t tile_a = tk * a.tiles_n + 2 * p;
            deepest = max(deepest, a.tile_max_lens[tile_a]);
            if (2 * p + 1 < a.tiles_n) deepest = max(deepest, a.tile_max_lens[tile_a + 1]);
        }
    }
    // (this kernel measures a little faster on 10 wavefronts with 204-byte lane strides -- 51 dwords, odd, so
    // the lanes' bytes spread over the banks -- than on 11 with 186: the shallow class is not used)
    const uint32_t cls = persist_classify(lds, a.tables, a.slot_map, deepest);
    if (cls == 2u)
        decode_wave_tiles<8, kDepthDeep, kMerge>(a, j, n_wg, tab, lds, wave, lane);
    else
        decode_wave_tiles<10, kDepthMedium, kMerge>(a, j, n_wg, tab, lds, wave, lane);
}

// Where an item lies: worked out once per item (the divisions are long instruction sequences) and handed on.
struct DecCoord {
    uint32_t item, hsel, seg, p, tk;
};
// ---- items of the sixteen-wavefront kernel, with what they read from memory asked for ahead ------------
// What an item reads before its window is known (requested two items ahead, looked at one item ahead) ...
struct DecRaw {
    uint32_t state, row, row_end;               // per lane, as stored (row: 0x7fffffff = from the body's last row)
    uint32_t off_a, depth_a, off_b, depth_b;    // the two tile bodies
};
// ... and the item ready to be staged.
struct DecItem {
    DecCoord co;
    uint32_t state;
    int32_t row;
    uint32_t w_lo, rows, win_a, win_b;  // first body row of the window, rows in it (both bodies / each)
    uint64_t base_a, base_b;
    bool fast;
};

__device__ __forceinline__ DecCoord dec_coord(const DecodeArgs &a, uint32_t item) {
    const uint32_t pairs = (a.tiles_n + 1) / 2;
    DecCoord c;
    c.item = item;
    c.hsel = item & 1u;
    const uint32_t us = item >> 1, pr = us / a.segs;
    c.seg = us - pr * a.segs;
    c.tk = pr / pairs;
    c.p = pr - c.tk * pairs;
    return c;
}

__device__ __forceinline__ void dec_request(const DecodeArgs &a, const DecCoord &co, int lane, DecRaw &m) {
    const uint32_t hsel = co.hsel, seg = co.seg, p = co.p, tk = co.tk;
    const uint32_t side = lane / 32, c = lane % 32;
    const bool have_b = 2 * p + 1 < a.tiles_n;
    const uint32_t tile_a = tk * a.tiles_n + 2 * p, tile_b = have_b ? tile_a + 1 : tile_a;
    m.off_a = a.tile_offsets[tile_a];
    m.depth_a = a.tile_max_lens[tile_a];
    m.off_b = a.tile_offsets[tile_b];
    m.depth_b = a.tile_max_lens[tile_b];
    const uint32_t tile = side ? tile_b : tile_a, q = hsel * 32 + c;
    const uint2 *ck = a.ckpt + ((size_t)tile * (a.segs - 1)) * 64 + q;  // (only read when segs > 1)
    if (seg == 0) {
        m.state = a.states[(size_t)tile * 64 + q];
        m.row = 0x7fffffffu;
    } else {
        const uint2 v = ck[(size_t)(seg - 1) * 64];
        m.state = v.x;
        m.row = v.y;
    }
    m.row_end = seg + 1 < a.segs ? ck[(size_t)seg * 64].y : 0xffffffffu;
}

// Same conditions as decode_one_item's.
template <bool kMerge>
__device__ __forceinline__ void dec_resolve(const DecodeArgs &a, const DecCoord &co, int lane, const DecRaw &m, DecItem &it) {
    const uint32_t hsel = co.hsel, seg = co.seg, p = co.p, tk = co.tk;
    const uint32_t half = a.th / 2, seglen = a.seglen, side = lane / 32, c = lane % 32;
    const uint32_t tn = 2 * p + side, col = tn * 32 + c, row_first = tk * a.th + hsel * half + seg * seglen;
    it.co = co;
    it.base_a = m.off_a;
    it.base_b = m.off_b;
    uint32_t depth_a = m.depth_a, depth_b = m.depth_b;
    if (it.base_a + (uint64_t)depth_a * 64 > a.stream_len) depth_a = 0;
    if (it.base_b + (uint64_t)depth_b * 64 > a.stream_len) depth_b = 0;
    const uint32_t depth = side ? depth_b : depth_a;
    it.state = m.state;
    it.row = min((int32_t)m.row, (int32_t)depth - 1);
    const int32_t row_end = min((int32_t)m.row_end, it.row);
    const bool col_ok = tn < a.tiles_n && col < a.N;
    const bool whole = row_first < a.K && a.K - row_first >= seglen;
    const int32_t w_lo = max(wave_min_i32(row_end) - 1, 0), w_hi = wave_max_i32(it.row);
    it.w_lo = (uint32_t)w_lo;
    it.win_a = (uint32_t)max(min(w_hi + 1, (int32_t)depth_a) - w_lo, 0);
    it.win_b = (uint32_t)max(min(w_hi + 1, (int32_t)depth_b) - w_lo, 0);
    it.rows = max(it.win_a, it.win_b);
    it.fast = __builtin_amdgcn_ballot_w64(!col_ok) == 0 && whole && it.win_a >= 2 && it.win_b >= 2 &&
              it.rows <= kDecWinRows && seglen % (kMerge ? 8 : 2) == 0 && seglen >= 2 &&
              (uint64_t)a.K * a.N < (1ull << (kMerge ? 31 : 32)) && (!kMerge || a.man_aligned);
}

// Touches the cache lines of the item's two windows (a 128-byte line per lane and body); the values are not
// used, the caller keeps them alive until the current item has been decoded.
__device__ __forceinline__ void dec_touch(const DecodeArgs &a, const DecItem &it, int lane, uint32_t &t, uint32_t &t2) {
    t = t2 = 0;
    if (!it.fast) return;
    if ((uint32_t)lane * 128 < it.win_a * 64)
        t = *reinterpret_cast<const uint32_t *>(a.stream + it.base_a + (size_t)it.w_lo * 64 + lane * 128);
    if ((uint32_t)lane * 128 < it.win_b * 64)
        t2 = *reinterpret_cast<const uint32_t *>(a.stream + it.base_b + (size_t)it.w_lo * 64 + lane * 128);
}

// A resolved, fast item: its window into the wavefront's area (before anything of the next item is asked
// for: loads complete in the order they were issued) ...
__device__ __forceinline__ void dec_stage(const DecodeArgs &a, const DecItem &it, uint8_t *stage, int lane) {
    stage_window_pair(stage, a.stream + it.base_a + (size_t)it.w_lo * 64, it.win_a,
                      a.stream + it.base_b + (size_t)it.w_lo * 64, it.win_b, it.co.hsel, it.rows, lane);
}

// ... then decode, store the exponent bytes.
__device__ __forceinline__ void dec_run(const DecodeArgs &a, const DecItem &it, uint8_t *stage, int lane) {
    const uint32_t hsel = it.co.hsel, seg = it.co.seg, p = it.co.p, tk = it.co.tk;
    const uint32_t half = a.th / 2, seglen = a.seglen, row_first = tk * a.th + hsel * half + seg * seglen;
    FastLane st;
    const int32_t rel = max(it.row - (int32_t)it.w_lo, -1);  // this lane's next byte, in rows of the window (-1: none left)
    st.X = it.state << 3;
    st.q = (uint32_t)(uintptr_t)stage + (uint32_t)(rel * 64 + lane);
    st.n1 = rel >= 0 ? stage[rel * 64 + lane] : 0;  // (a wavefront's LDS operations complete in order)
    const uint64_t ob = reinterpret_cast<uint64_t>(a.out_exp + (size_t)row_first * a.N + 2 * p * 32);
    // readfirstlane returns a signed int: widen through uint32_t
    const uint32_t ob_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(ob >> 32));
    const uint32_t ob_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)ob);
    decode_tile_asm(st, ((uint64_t)ob_hi << 32) | (uint64_t)ob_lo, lane, a.N, seglen / 2, 64);
}

// The same batch on sixteen wavefronts per workgroup, for tensors whose items are short (see kDecSegWaves).
// A wavefront walks its items with the next one's checkpoints requested and its windows touched before the
// current one is decoded; an item whose window turns out larger than its area, a ragged one, and every item
// of a merging decode take decode_one_item.
template <bool kMerge>
__global__ __launch_bounds__(kDecSegWaves *kWave) void decode_tiled32_seg_kernel(DecodeBatchArgs b) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    uint32_t i = 0;
    while (i + 1 < b.n && blockIdx.x >= b.first_block[i + 1]) ++i;
    // (a copy: the tensor's description then sits in scalar registers, where a reference into the kernel
    // arguments at a variable index would be read from memory again wherever a field is used)
    const DecodeArgs a = b.item[i];
    const uint32_t j = blockIdx.x - b.first_block[i], n_wg = b.first_block[i + 1] - b.first_block[i];
    const uint64_t n_units = decode_num_pairs(a) * a.segs;  // unit = one segment of a pair, both halves
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kDecWinBytes;
    // this wavefront's items: slot = wave, wave + 16, ...; slot / 2 picks the workgroup's unit, slot % 2 the half
    auto item_of = [&](uint32_t slot, uint32_t &item) {
        const uint64_t unit = (uint64_t)(slot >> 1) * n_wg + j;
        item = (uint32_t)unit * 2 + (slot & 1u);
        return unit < n_units;
    };
    if (kMerge) {
        build_slot_table_x8(reinterpret_cast<uint2 *>(lds), a.tables, a.slot_map, tid, kDecSegWaves * kWave);
        __syncthreads();
        uint32_t item;
        for (uint32_t slot = wave; item_of(slot, item); slot += kDecSegWaves)
            decode_one_item<0, true>(a, item, tab, stage, lane);
        return;
    }
    DecRaw raw;
    DecItem nxt;
    nxt.fast = false;
    uint32_t slot = wave, item_n = 0, item_nn = 0;
    bool have_n = item_of(slot, item_n), have_nn = false;
    DecCoord co_n = dec_coord(a, item_n), co_nn = co_n;
    if (have_n) dec_request(a, co_n, lane, raw);  // on its way while the table is built
    build_slot_table_x8(reinterpret_cast<uint2 *>(lds), a.tables, a.slot_map, tid, kDecSegWaves * kWave);
    if (have_n) {
        dec_resolve<false>(a, co_n, lane, raw, nxt);
        have_nn = item_of(slot + kDecSegWaves, item_nn);
        if (have_nn) {
            co_nn = dec_coord(a, item_nn);
            dec_request(a, co_nn, lane, raw);
        }
    }
    __syncthreads();
    while (have_n) {
        const DecItem cur = nxt;
        if (cur.fast) dec_stage(a, cur, stage, lane);
        uint32_t touched = 0, touched2 = 0;
        have_n = have_nn;
        co_n = co_nn;
        slot += kDecSegWaves;
        if (have_n) {
            dec_resolve<false>(a, co_n, lane, raw, nxt);
            dec_touch(a, nxt, lane, touched, touched2);
            have_nn = item_of(slot + kDecSegWaves, item_nn);
            if (have_nn) {
                co_nn = dec_coord(a, item_nn);
                dec_request(a, co_nn, lane, raw);
            }
        }
        if (cur.fast)
            dec_run(a, cur, stage, lane);
        else
            decode_one_item<0, false>(a, cur.co.item, tab, stage, lane);
        asm volatile("" ::"v"(touched), "v"(touched2));  // the touching loads end here
    }
}


// Any tile width: one thread per stream, bytes read where they lie.  Used for widths other
// than 32 (the reference's tests sweep 16..128, tests/test_mat_mul.py:263-264) and, with kHalves = 1, for
// the layout of one stream per column and tile (comp_inference/rans_triton.py:399-464).
template <bool kMerge, uint32_t kHalves>
__global__ __launch_bounds__(256) void decode_tiled_generic_kernel(DecodeArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    const uint32_t spt = kHalves * a.tw;
    const uint64_t sid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (sid >= (uint64_t)a.num_tiles * spt) return;
    const uint32_t tile = (uint32_t)(sid / spt), q = (uint32_t)(sid % spt);
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t half = a.th / kHalves, hsel = q / a.tw, c = q % a.tw;
    const uint32_t col = tn * a.tw + c, my_row0 = tk * a.th + hsel * half;
    if (col >= a.N || my_row0 >= a.K) return;
    const uint32_t my_steps = min(half, a.K - my_row0);
    uint64_t base = a.tile_offsets[tile];
    uint32_t depth = a.tile_max_lens[tile];
    if (base + (uint64_t)depth * spt > a.stream_len) depth = 0;
    GlobalBytes src;
    src.init(a.stream + base, depth, spt, q);
    uint32_t x = a.states[sid];
    const uint8_t *man = kMerge ? a.man_tiled + (size_t)tile * a.th * a.tw + (size_t)hsel * half * a.tw + c
                                : nullptr;
    for (uint32_t i = 0; i < my_steps; ++i) {
        uint32_t sym = decode_symbol(x, tab) >> 24;
        src.renorm(x);
        src.renorm(x);
        size_t o = (size_t)(my_row0 + i) * a.N + col;
        if (kMerge)
            a.out_bf16[o] = (uint16_t)assemble_bf16(sym, man[(size_t)i * a.tw]);
        else
            a.out_exp[o] = (uint8_t)sym;
    }
}

// Decoder checkpoints.  A stream is a chain of th/2 dependent steps; with the decoder's state and
// byte position recorded at `segs` evenly spaced rows, the segments of a stream can be decoded by
// different wavefronts at the same time.  The checkpoints are derived from the stream (an index kept
// beside it), the stream itself is untouched.  One thread per stream walks it once:
// ckpt[(tile * (segs - 1) + j - 1) * 2 tw + q] = {state, row of the next unread byte (-1: none left)}
// at the first row of segment j = 1 .. segs - 1 of stream q.  The reference keeps such checkpoints for
// its flat format only (src/cuda/rans_kernels.cuh:454-465).
__global__ __launch_bounds__(256) void checkpoints_kernel(DecodeArgs a, uint32_t segs, uint2 *__restrict__ ckpt) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    const uint32_t spt = 2 * a.tw;
    const uint64_t sid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (sid >= (uint64_t)a.num_tiles * spt) return;
    const uint32_t tile = (uint32_t)(sid / spt), q = (uint32_t)(sid % spt);
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t half = a.th / 2, seglen = half / segs, hsel = q / a.tw, c = q % a.tw;
    const uint32_t col = tn * a.tw + c, my_row0 = tk * a.th + hsel * half;
    const uint32_t my_steps = (col < a.N && my_row0 < a.K) ? min(half, a.K - my_row0) : 0u;
    uint64_t base = a.tile_offsets[tile];
    uint32_t depth = a.tile_max_lens[tile];
    if (base + (uint64_t)depth * spt > a.stream_len) depth = 0;
    GlobalBytes src;
    src.init(a.stream + base, depth, spt, q);
    uint32_t x = a.states[sid];
    uint2 *mine = ckpt + (size_t)tile * (segs - 1) * spt + q;
    uint32_t next = 1;
    for (uint32_t i = 0; i < my_steps; ++i) {
        if (next < segs && i == next * seglen) {
            mine[(size_t)(next - 1) * spt] = make_uint2(x, (uint32_t)src.row);
            ++next;
        }
        decode_symbol(x, tab);
        src.renorm(x);
        src.renorm(x);
    }
    for (; next < segs; ++next) mine[(size_t)(next - 1) * spt] = make_uint2(x, (uint32_t)src.row);  // short streams
}

}  // namespace ci

using namespace ci;

extern "C" size_t ci_checkpoint_bytes(uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width,
                                      uint32_t segments) {
    if (tile_height == 0 || tile_width == 0 || segments < 2) return 0;
    return (size_t)ceil_div(K, tile_height) * ceil_div(N, tile_width) * (segments - 1) * 2 * tile_width * sizeof(uint2);
}

extern "C" int ci_build_checkpoints_ilp2(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                         const uint32_t *d_tables, const uint8_t *d_slot_map,
                                         const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens, uint32_t K,
                                         uint32_t N, uint32_t tile_height, uint32_t tile_width, uint32_t segments,
                                         void *d_checkpoints, size_t checkpoint_bytes, ci_stream_t stream) {
    if (K == 0 || N == 0 || segments < 2) return CI_OK;
    if (!d_states || !d_tables || !d_slot_map || !d_tile_offsets || !d_tile_max_lens || !d_checkpoints)
        return fail(CI_ERR_ARG, "ci_build_checkpoints_ilp2: null pointer");
    if (stream_len && !d_stream) return fail(CI_ERR_ARG, "ci_build_checkpoints_ilp2: null stream");
    if (tile_height == 0 || tile_width == 0 || (tile_height & 1) || (tile_height / 2) % segments)
        return fail(CI_ERR_ARG, "ci_build_checkpoints_ilp2: half the tile height must be a multiple of the segment count");
    if (!aligned(d_slot_map, 4) || !aligned(d_checkpoints, 8))
        return fail(CI_ERR_ARG, "ci_build_checkpoints_ilp2: slot_map must be 4-byte, checkpoints 8-byte aligned");
    const size_t need = ci_checkpoint_bytes(K, N, tile_height, tile_width, segments);
    if (checkpoint_bytes < need)
        return fail(CI_ERR_CAPACITY, "ci_build_checkpoints_ilp2: checkpoints need %zu bytes, got %zu", need, checkpoint_bytes);
    DecodeArgs a = {};
    a.stream = d_stream;
    a.stream_len = stream_len;
    a.states = d_states;
    a.tables = d_tables;
    a.slot_map = d_slot_map;
    a.tile_offsets = d_tile_offsets;
    a.tile_max_lens = d_tile_max_lens;
    a.K = K;
    a.N = N;
    a.th = tile_height;
    a.tw = tile_width;
    a.tiles_n = ceil_div(N, tile_width);
    a.num_tiles = ceil_div(K, tile_height) * a.tiles_n;
    const uint64_t streams = (uint64_t)a.num_tiles * 2 * tile_width;
    hipLaunchKernelGGL(checkpoints_kernel, dim3((uint32_t)((streams + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a, segments, static_cast<uint2 *>(d_checkpoints));
    CI_LAUNCH_CHECK("checkpoints_kernel");
    return CI_OK;
}

// Segmented decode: 32-column tiles whose half height splits into `segments` runs of whole 16-row blocks.
static int check_segments(const char *who, uint32_t tile_height, uint32_t segments, const void *d_checkpoints) {
    if (tile_height % 2 || (tile_height / 2) % (16 * segments))
        return fail(CI_ERR_ARG, "%s: %u segments need a tile half height that is a multiple of %u", who, segments,
                    16 * segments);
    if (!d_checkpoints || !aligned(d_checkpoints, 8))
        return fail(CI_ERR_ARG, "%s: segments without (8-byte aligned) checkpoints", who);
    return CI_OK;
}

// Launch the persistent kernel over the (already checked) tensors of `b`: the device's CUs are
// divided among the tensors in proportion to their tile counts.
// Rows of the longest item the sixteen-wavefront kernel is given (bf16 weight exponents take about a third
// of a byte per symbol and the lanes of a tile drift apart by some twenty rows: 256 rows stay below the
// window area; an item whose window is larger takes the guarded path).
constexpr uint32_t kDecSegRows = 256;

static int launch_persist(DecodeBatchArgs &b, bool merge, hipStream_t s) {
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    // The unit handed to a workgroup is a pair of neighbouring column tiles, or one segment of it.
    uint64_t pairs[kDecBatchMax], total = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        const DecodeArgs &a = b.item[i];
        pairs[i] = (uint64_t)(a.num_tiles / a.tiles_n) * ((a.tiles_n + 1) / 2) * a.segs;
        total += pairs[i];
    }
    // Never more workgroups than CUs (one is resident per CU; a workgroup too many would run alone
    // after all the others): floor of the proportional share, then hand out what is left to the
    // tensors with the most pairs per workgroup.
    uint32_t share[kDecBatchMax], used = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        uint64_t sh = pairs[i] * cus / total;  // total >= 1: empty tensors are not in b
        sh = sh < 1 ? 1 : sh;
        share[i] = (uint32_t)(sh > pairs[i] ? pairs[i] : sh);
        used += share[i];
    }
    while (used < cus) {
        int best = -1;
        for (uint32_t i = 0; i < b.n; ++i)
            if (share[i] < pairs[i] && (best < 0 || pairs[i] * share[best] > pairs[best] * share[i])) best = (int)i;
        if (best < 0) break;  // every tensor already has one workgroup per pair
        ++share[best];
        ++used;
    }
    uint32_t blocks = 0;
    for (uint32_t i = 0; i < b.n; ++i) {
        b.first_block[i] = blocks;
        blocks += share[i];
    }
    b.first_block[b.n] = blocks;
    // Items of at most kDecSegRows rows (segments of streams, or low tiles) have windows that fit 7 KB: such a
    // batch runs on sixteen wavefronts per CU.
    bool short_items = true;
    for (uint32_t i = 0; i < b.n; ++i) short_items = short_items && b.item[i].th / 2 / b.item[i].segs <= kDecSegRows;
    const dim3 grid(blocks);
    if (short_items) {
        CI_ALLOW_FULL_LDS(decode_tiled32_seg_kernel<false>);
        CI_ALLOW_FULL_LDS(decode_tiled32_seg_kernel<true>);
        const dim3 block(kDecSegWaves * kWave);
        const uint32_t lds_bytes = kSlotTableBytes + kDecSegWaves * kDecWinBytes;
        if (merge)
            hipLaunchKernelGGL(decode_tiled32_seg_kernel<true>, grid, block, lds_bytes, s, b);
        else
            hipLaunchKernelGGL(decode_tiled32_seg_kernel<false>, grid, block, lds_bytes, s, b);
        CI_LAUNCH_CHECK("decode_tiled32_seg_kernel");
        return CI_OK;
    }
    CI_ALLOW_FULL_LDS(decode_tiled32_persist_kernel<false>);
    CI_ALLOW_FULL_LDS(decode_tiled32_persist_kernel<true>);
    const dim3 block(kPersistWaves * kWave);
    if (merge)
        hipLaunchKernelGGL(decode_tiled32_persist_kernel<true>, grid, block, kLdsLimit, s, b);
    else
        hipLaunchKernelGGL(decode_tiled32_persist_kernel<false>, grid, block, kLdsLimit, s, b);
    CI_LAUNCH_CHECK("decode_tiled32_persist_kernel");
    return CI_OK;
}

extern "C" int ci_decode_tiled_ilp2_batch(const ci_decode_item *h_items, uint32_t n_items, ci_stream_t stream) {
    if (n_items == 0) return CI_OK;
    if (!h_items) return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2_batch: null item list");
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t done = 0;
    while (done < n_items) {
        DecodeBatchArgs b;
        b.n = 0;
        for (; done < n_items && b.n < (uint32_t)kDecBatchMax; ++done) {
            const ci_decode_item &it = h_items[done];
            if (it.K == 0 || it.N == 0) continue;
            // items the batched kernel cannot take go through the single-tensor entry point
            if (it.tile_width != 32 || !aligned(it.d_stream, 16)) {
                int rc = ci_decode_tiled_ilp2(it.d_stream, it.stream_len, it.d_states, it.d_tables, it.d_slot_map,
                                              it.d_tile_offsets, it.d_tile_max_lens, it.K, it.N, it.tile_height,
                                              it.tile_width, it.d_out_exp, nullptr, nullptr, stream);
                if (rc) return rc;
                continue;
            }
            if (!it.d_states || !it.d_tables || !it.d_slot_map || !it.d_tile_offsets || !it.d_tile_max_lens ||
                !it.d_out_exp || (it.stream_len && !it.d_stream))
                return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2_batch: null pointer in item %u", done);
            if (it.tile_height == 0 || (it.tile_height & 1) || !aligned(it.d_slot_map, 4))
                return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2_batch: bad tile height or slot_map alignment in item %u", done);
            DecodeArgs &a = b.item[b.n];
            a.stream = it.d_stream;
            a.stream_len = it.stream_len;
            a.states = it.d_states;
            a.tables = it.d_tables;
            a.slot_map = it.d_slot_map;
            a.tile_offsets = it.d_tile_offsets;
            a.tile_max_lens = it.d_tile_max_lens;
            a.K = it.K;
            a.N = it.N;
            a.th = it.tile_height;
            a.tw = 32;
            a.tiles_n = ceil_div(it.N, 32);
            a.num_tiles = ceil_div(it.K, it.tile_height) * a.tiles_n;
            a.out_exp = it.d_out_exp;
            a.man_tiled = nullptr;
            a.out_bf16 = nullptr;
            a.man_aligned = 0;
            a.ckpt = nullptr;
            a.segs = 1;
            a.seglen = it.tile_height / 2;
            if (it.segments > 1) {
                if (int rc = check_segments("ci_decode_tiled_ilp2_batch", it.tile_height, it.segments, it.d_checkpoints))
                    return rc;
                a.ckpt = static_cast<const uint2 *>(it.d_checkpoints);
                a.segs = it.segments;
                a.seglen = it.tile_height / 2 / it.segments;
            }
            ++b.n;
        }
        if (b.n == 0) continue;
        if (int rc = launch_persist(b, false, s)) return rc;
    }
    return CI_OK;
}

extern "C" int ci_decode_tiled_ilp2(const uint8_t *d_stream, uint64_t stream_len,
                                    const uint32_t *d_states, const uint32_t *d_tables,
                                    const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                    const uint32_t *d_tile_max_lens, uint32_t K, uint32_t N,
                                    uint32_t tile_height, uint32_t tile_width, uint8_t *d_out_exp,
                                    const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                                    ci_stream_t stream) {
    return ci_decode_tiled_ilp2_segmented(d_stream, stream_len, d_states, d_tables, d_slot_map, d_tile_offsets,
                                          d_tile_max_lens, K, N, tile_height, tile_width, nullptr, 1, d_out_exp,
                                          d_man_tiled, d_out_bf16, stream);
}

extern "C" int ci_decode_tiled_ilp2_segmented(const uint8_t *d_stream, uint64_t stream_len,
                                              const uint32_t *d_states, const uint32_t *d_tables,
                                              const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                              const uint32_t *d_tile_max_lens, uint32_t K, uint32_t N,
                                              uint32_t tile_height, uint32_t tile_width,
                                              const void *d_checkpoints, uint32_t segments, uint8_t *d_out_exp,
                                              const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                                              ci_stream_t stream) {
    if (K == 0 || N == 0) return CI_OK;
    if (!d_states || !d_tables || !d_slot_map || !d_tile_offsets || !d_tile_max_lens)
        return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: null table or metadata pointer");
    if (stream_len && !d_stream) return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: null stream");
    if (tile_height == 0 || tile_width == 0 || (tile_height & 1))
        return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: tile_height must be even and non-zero");
    const bool merge = d_man_tiled != nullptr;
    if (merge && !d_out_bf16) return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: merge asked without bf16 output");
    if (!merge && !d_out_exp) return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: null output");
    if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "ci_decode_tiled_ilp2: slot_map must be 4-byte aligned");

    DecodeArgs a;
    a.stream = d_stream;
    a.stream_len = stream_len;
    a.states = d_states;
    a.tables = d_tables;
    a.slot_map = d_slot_map;
    a.tile_offsets = d_tile_offsets;
    a.tile_max_lens = d_tile_max_lens;
    a.K = K;
    a.N = N;
    a.th = tile_height;
    a.tw = tile_width;
    a.tiles_n = ceil_div(N, tile_width);
    a.num_tiles = ceil_div(K, tile_height) * a.tiles_n;
    a.out_exp = d_out_exp;
    a.man_tiled = d_man_tiled;
    a.out_bf16 = d_out_bf16;
    hipStream_t s = static_cast<hipStream_t>(stream);

    a.man_aligned = merge && aligned(d_man_tiled, 4) ? 1u : 0u;
    a.ckpt = nullptr;
    a.segs = 1;
    a.seglen = tile_height / 2;
    if (segments > 1 && tile_width == 32) {  // (other widths decode one thread per stream: nothing to split)
        if (int rc = check_segments("ci_decode_tiled_ilp2_segmented", tile_height, segments, d_checkpoints)) return rc;
        a.ckpt = static_cast<const uint2 *>(d_checkpoints);
        a.segs = segments;
        a.seglen = tile_height / 2 / segments;
    }
    if (tile_width == 32 && aligned(d_stream, 16)) {
        DecodeBatchArgs b;
        b.n = 1;
        b.item[0] = a;
        if (int rc = launch_persist(b, merge, s)) return rc;
    } else {
        const uint64_t streams = (uint64_t)a.num_tiles * 2 * tile_width;
        const dim3 grid((uint32_t)((streams + 255) / 256)), block(256);
        if (merge)
            hipLaunchKernelGGL((decode_tiled_generic_kernel<true, 2>), grid, block, 0, s, a);
        else
            hipLaunchKernelGGL((decode_tiled_generic_kernel<false, 2>), grid, block, 0, s, a);
        CI_LAUNCH_CHECK("decode_tiled_generic_kernel");
    }
    return CI_OK;
}

extern "C" int ci_decode_tiled_one(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                   const uint32_t *d_tables, const uint8_t *d_slot_map,
                                   const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens, uint32_t K,
                                   uint32_t N, uint32_t tile_height, uint32_t tile_width, uint8_t *d_out_exp,
                                   const uint8_t *d_man_tiled, uint16_t *d_out_bf16, ci_stream_t stream) {
    if (K == 0 || N == 0) return CI_OK;
    if (!d_states || !d_tables || !d_slot_map || !d_tile_offsets || !d_tile_max_lens)
        return fail(CI_ERR_ARG, "ci_decode_tiled_one: null table or metadata pointer");
    if (stream_len && !d_stream) return fail(CI_ERR_ARG, "ci_decode_tiled_one: null stream");
    if (tile_height == 0 || tile_width == 0) return fail(CI_ERR_ARG, "ci_decode_tiled_one: empty tile");
    const bool merge = d_man_tiled != nullptr;
    if (merge ? !d_out_bf16 : !d_out_exp) return fail(CI_ERR_ARG, "ci_decode_tiled_one: null output");
    if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "ci_decode_tiled_one: slot_map must be 4-byte aligned");
    DecodeArgs a;
    a.stream = d_stream;
    a.stream_len = stream_len;
    a.states = d_states;
    a.tables = d_tables;
    a.slot_map = d_slot_map;
    a.tile_offsets = d_tile_offsets;
    a.tile_max_lens = d_tile_max_lens;
    a.K = K;
    a.N = N;
    a.th = tile_height;
    a.tw = tile_width;
    a.tiles_n = ceil_div(N, tile_width);
    a.num_tiles = ceil_div(K, tile_height) * a.tiles_n;
    a.out_exp = d_out_exp;
    a.man_tiled = d_man_tiled;
    a.out_bf16 = d_out_bf16;
    a.man_aligned = 0;
    a.ckpt = nullptr;
    a.segs = 1;
    a.seglen = tile_height;
    const uint64_t streams = (uint64_t)a.num_tiles * tile_width;
    const dim3 grid((uint32_t)((streams + 255) / 256)), block(256);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (merge)
        hipLaunchKernelGGL((decode_tiled_generic_kernel<true, 1>), grid, block, 0, s, a);
    else
        hipLaunchKernelGGL((decode_tiled_generic_kernel<false, 1>), grid, block, 0, s, a);
    CI_LAUNCH_CHECK("decode_tiled_generic_kernel");
    return CI_OK;
}

extern "C" int ci_decode_tiled(const ci_tiled_weight *w, uint8_t *d_out_exp, uint16_t *d_out_bf16, ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (d_out_bf16 && !w->d_man_tiled) return fail(CI_ERR_ARG, "ci_decode_tiled: bf16 asked of a weight without sign|mantissa plane");
    const uint32_t segments = w->segments > 1 ? w->segments : 1;
    return ci_decode_tiled_ilp2_segmented(w->d_stream, w->stream_len, w->d_states, w->d_tables, w->d_slot_map,
                                          w->d_tile_offsets, w->d_tile_max_lens, w->K, w->N, w->tile_height,
                                          w->tile_width, segments > 1 ? w->d_checkpoints : nullptr, segments,
                                          d_out_bf16 ? nullptr : d_out_exp, d_out_bf16 ? w->d_man_tiled : nullptr,
                                          d_out_bf16, stream);
}
