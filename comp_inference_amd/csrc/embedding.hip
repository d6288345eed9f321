// Fused decompress + gather (embedding lookup) on gfx950.
//
// out[t, :] = table[ids[t], :] for a table stored as rANS-coded exponent plane + raw
// sign|mantissa plane; ids outside [0, K) give zero rows.  Replaces
// fused_rans_embedding_triton / fused_rans_embedding_kernel_ilp2
// (comp_inference/embedding_triton.py:170-330) and the dense-layout variant (:333-483).
//
// The reference starts one program per (token, column tile) and discards row % (th/2) decode
// steps in each.  Here the ids are first grouped by "bucket" (one workgroup: counting, or a bitonic
// sort for tables with more buckets than the counters hold); a bucket is one half tile of rows, i.e.
// the row range of one stream.  A work item is one bucket of two neighbouring column tiles (32 + 32
// lanes, all on the same half): a wavefront walks the two half tiles once up to the deepest requested
// row and writes every requested row on the way as one 128-byte store.  Items of buckets nobody
// asked for are skipped before touching the stream.
// With decoder checkpoints (ci_build_checkpoints_ilp2) a bucket is one *segment* of a half tile: the
// walk starts at the segment's checkpoint instead of the top of the stream, so a requested row costs at
// most th / (2 segments) decode steps instead of th / 2.
#include "ci_common.h"
#include "rans_device.h"
#include "fast_tile.h"

namespace ci {

constexpr uint32_t kEmbChunk = 8192;  // ids sorted per pass (64 KB of LDS)
constexpr uint32_t kEmbRun = 64;      // most requests one wavefront serves for one bucket

__host__ __device__ inline uint32_t emb_max_chunks(uint32_t n_ids, uint32_t n_buckets) {
    const uint32_t by_bucket = n_ids < n_buckets + 1 ? n_ids : n_buckets + 1;
    return n_ids / kEmbRun + by_bucket + 1;
}

struct EmbedArgs {
    const int64_t *ids;
    uint32_t n_ids;
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
    uint32_t K, N, th, tw, tiles_n, n_buckets;
    const uint2 *ckpt;     // decoder checkpoints, or null
    uint32_t segs;         // segments per stream (1 without checkpoints)
    uint32_t bucket_rows;  // rows of a bucket: th / (2 segs)
    uint16_t *out;
    uint32_t out_stride;
    uint32_t *keys;          // workspace: sorted row ids (invalid = 0xFFFFFFFF, sorted last)
    uint32_t *pos;           // workspace: output row of each sorted id
    uint2 *chunk_rec;        // workspace: per chunk {first sorted request, its key}, then {n_ids, -}; the word at
                             // chunk_count holds the number of chunks (bucket n_buckets collects the invalid ids)
    uint32_t *chunk_count;
    uint32_t n_pad;          // n_ids rounded up to a power of two
};

// Keys below this many rows and positions below kEmbChunk fit one word.
constexpr uint32_t kEmbPosBits = 13, kEmbPackedInvalid = (1u << (32 - kEmbPosBits)) - 1;
static_assert((1u << kEmbPosBits) == kEmbChunk, "a position inside a pass must fit its bit field");

// One workgroup: sort (id, position) by id, then list the chunks of requests.  kPacked: while the row
// ids fit 19 bits an element of the sort is one word, id << 13 | position (the same order as the pair,
// ties included), which halves the LDS traffic and the instructions of a compare-exchange -- and one CU
// does all of this work.
template <bool kPacked>
__global__ __launch_bounds__(1024) void embed_sort_kernel(EmbedArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t *key = reinterpret_cast<uint32_t *>(lds);
    uint32_t *val = key + a.n_pad;
    const uint32_t tid = threadIdx.x, half = a.bucket_rows;  // rows of a bucket
    for (uint32_t i = tid; i < a.n_pad; i += 1024) {
        uint32_t k = kPacked ? kEmbPackedInvalid : 0xFFFFFFFFu;  // invalid ids sort last
        if (i < a.n_ids) {
            const int64_t id = a.ids[i];
            if (id >= 0 && id < (int64_t)a.K) k = (uint32_t)id;
        }
        key[i] = kPacked ? (k << kEmbPosBits) | i : k;
        if (!kPacked) val[i] = i;
    }
    __syncthreads();
    // Compare-exchange t works on elements inside the aligned block of 2 * stride elements that holds 2 t.  For
    // strides up to 64 the 64 exchanges of a wavefront stay inside that wavefront's own 128 elements (and
    // exchange t belongs to the same thread in every stage), so those stages need no workgroup barrier:
    // the LDS serves one wavefront's accesses in order.  Barriers remain around the stages with longer
    // strides -- 14 instead of 66 for 2048 ids.
    for (uint32_t size = 2; size <= a.n_pad; size <<= 1)
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t t = tid; t < a.n_pad / 2; t += 1024) {
                const uint32_t lo = 2 * t - (t & (stride - 1)), hi = lo + stride;
                const bool up = (lo & size) == 0;
                const uint32_t ka = key[lo], kb = key[hi];
                if (kPacked) {
                    if ((ka > kb) == up) {
                        key[lo] = kb;
                        key[hi] = ka;
                    }
                } else {
                    const uint32_t va = val[lo], vb = val[hi];
                    // ties are ordered by position so that the result does not depend on the network
                    const bool gt = ka > kb || (ka == kb && va > vb);
                    if (gt == up) {
                        key[lo] = kb;
                        key[hi] = ka;
                        val[lo] = vb;
                        val[hi] = va;
                    }
                }
            }
            // the stage that follows: stride / 2, or size (the first of the next size) after stride 1
            const uint32_t next_stride = stride > 1 ? stride >> 1 : size;
            if (stride > 64 || next_stride > 64) {
                __syncthreads();
            } else {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
        }
    __syncthreads();
    if (kPacked) {  // back to (id, position) for what follows
        uint32_t e[kEmbChunk / 1024];
#pragma unroll
        for (uint32_t r = 0; r < kEmbChunk / 1024; ++r) e[r] = tid + 1024 * r < a.n_pad ? key[tid + 1024 * r] : 0u;
#pragma unroll
        for (uint32_t r = 0; r < kEmbChunk / 1024; ++r) {
            const uint32_t i = tid + 1024 * r;
            if (i < a.n_pad) {
                const uint32_t id = e[r] >> kEmbPosBits;
                key[i] = id == kEmbPackedInvalid ? 0xFFFFFFFFu : id;
                val[i] = e[r] & (kEmbChunk - 1);
            }
        }
        __syncthreads();
    }
    for (uint32_t i = tid; i < a.n_ids; i += 1024) {
        a.keys[i] = key[i];
        a.pos[i] = val[i];
    }
    // Chunks: runs of sorted requests of one bucket, cut at every multiple of kEmbRun, so that a
    // bucket many ids fall into is served by several wavefronts.  Request i opens a chunk if it is
    // the first of its bucket or i is a multiple of kEmbRun; the chunk list is the compaction of
    // those i: each thread counts its own consecutive requests, a scan over the counts gives the
    // offsets.
    auto bucket_of = [&](uint32_t i) { return key[i] == 0xFFFFFFFFu ? a.n_buckets : key[i] / half; };
    auto opens = [&](uint32_t i) {
        return i < a.n_ids && (i == 0 || i % kEmbRun == 0 || bucket_of(i) != bucket_of(i - 1));
    };
    uint32_t *wave_total = key + 2 * a.n_pad;  // 16 counters behind the two sort arrays
    const uint32_t per = (a.n_pad + 1023) / 1024;
    uint32_t mine = 0;
    for (uint32_t u = 0; u < per; ++u) mine += opens(tid * per + u) ? 1u : 0u;
    // inclusive scan inside the wavefront, then over the 16 wavefront totals
    uint32_t incl = mine;
    const uint32_t lane = tid % 64, wv = tid / 64;
#pragma unroll
    for (uint32_t d = 1; d < 64; d <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, d, 64);
        if (lane >= d) incl += up;
    }
    if (lane == 63) wave_total[wv] = incl;
    __syncthreads();
    uint32_t before = 0, total = 0;
    for (uint32_t w = 0; w < 16; ++w) {
        const uint32_t t = wave_total[w];
        if (w < wv) before += t;
        total += t;
    }
    uint32_t at = before + incl - mine;
    for (uint32_t u = 0; u < per; ++u) {
        const uint32_t i = tid * per + u;
        if (opens(i)) a.chunk_rec[at++] = make_uint2(i, key[i]);
    }
    if (tid == 0) {
        a.chunk_rec[total] = make_uint2(a.n_ids, 0xFFFFFFFFu);  // end marker
        *a.chunk_count = total;
    }
}

// The same lists by counting instead of sorting, for tables of up to kGroupMaxSlots counting slots: the
// gather needs its requests grouped by bucket, and in row order only inside a chunk, which the wavefront
// that serves the chunk establishes itself (sort_chunk_rows).  A slot is a run of `fine_rows` rows (a
// divisor of the bucket's rows, 1 for small tables): one pass counts the requests of every slot (LDS
// atomics; the value returned is the request's rank in its slot), a scan gives every slot its first
// position, the buckets' request counts follow from the slots' positions, a second scan gives every
// bucket its first chunk, and a last pass scatters.  Requests thus lie in slot order -- the chunks of a
// bucket many ids fall into cover ascending row ranges, as after a sort -- and in the order the atomics
// came inside a slot, which changes from run to run; the gathered rows do not.
constexpr uint32_t kGroupMaxSlots = 16384;  // two words of LDS per slot

// Exclusive prefix of `mine` over the 1024 threads (via 16 wavefront totals in `wave_sum`); `total` = the sum.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t mine, uint32_t *wave_sum, uint32_t tid, uint32_t &total) {
    const uint32_t lane = tid % 64, wv = tid / 64;
    uint32_t incl = mine;
#pragma unroll
    for (uint32_t d = 1; d < 64; d <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, d, 64);
        if (lane >= d) incl += up;
    }
    __syncthreads();  // (wave_sum may still be read from an earlier scan)
    if (lane == 63) wave_sum[wv] = incl;
    __syncthreads();
    uint32_t before = incl - mine;
    total = 0;
    for (uint32_t w = 0; w < 16; ++w) {
        const uint32_t t = wave_sum[w];
        if (w < wv) before += t;
        total += t;
    }
    return before;
}

__global__ __launch_bounds__(1024) void embed_group_kernel(EmbedArgs a, uint32_t fine_rows) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t nf = (a.K + fine_rows - 1) / fine_rows;  // slots of valid rows; slot nf collects the invalid ids
    const uint32_t per_bucket = a.bucket_rows / fine_rows;  // slots of a bucket
    uint32_t *cnt = reinterpret_cast<uint32_t *>(lds), *first = cnt + (nf + 1), *wave_sum = first + (nf + 2);
    const uint32_t tid = threadIdx.x;
    for (uint32_t f = tid; f <= nf; f += 1024) cnt[f] = 0;
    __syncthreads();
    uint32_t key[kEmbChunk / 1024], slot[kEmbChunk / 1024], rank[kEmbChunk / 1024];
#pragma unroll
    for (uint32_t r = 0; r < kEmbChunk / 1024; ++r) {
        const uint32_t i = tid + 1024 * r;
        key[r] = 0xFFFFFFFFu;
        slot[r] = nf;
        rank[r] = 0;
        if (i < a.n_ids) {
            const int64_t id = a.ids[i];
            if (id >= 0 && id < (int64_t)a.K) {
                key[r] = (uint32_t)id;
                slot[r] = key[r] / fine_rows;
            }
            rank[r] = atomicAdd(&cnt[slot[r]], 1u);
        }
    }
    __syncthreads();
    // first position of every slot: every thread takes a run of neighbouring slots
    {
        const uint32_t per = (nf + 1 + 1023) / 1024, f0 = min(tid * per, nf + 1), f1 = min(f0 + per, nf + 1);
        uint32_t mine = 0, total;
        for (uint32_t f = f0; f < f1; ++f) mine += cnt[f];
        uint32_t at = block_exclusive_scan(mine, wave_sum, tid, total);
        for (uint32_t f = f0; f < f1; ++f) {
            first[f] = at;
            at += cnt[f];
        }
        if (tid == 0) first[nf + 1] = total;
    }
    __syncthreads();
    // chunks: every thread takes a run of neighbouring buckets (bucket n_buckets = the invalid ids)
    {
        const uint32_t nb1 = a.n_buckets + 1, per = (nb1 + 1023) / 1024, b0 = min(tid * per, nb1), b1 = min(b0 + per, nb1);
        auto span = [&](uint32_t b, uint32_t &lo, uint32_t &n) {  // the bucket's requests: positions lo .. lo + n
            const uint32_t fa = b == a.n_buckets ? nf : min(b * per_bucket, nf);
            const uint32_t fb = b == a.n_buckets ? nf + 1 : min((b + 1) * per_bucket, nf);
            lo = first[fa];
            n = first[fb] - lo;
        };
        uint32_t mine = 0, total;
        for (uint32_t b = b0; b < b1; ++b) {
            uint32_t lo, n;
            span(b, lo, n);
            mine += (n + kEmbRun - 1) / kEmbRun;
        }
        uint32_t at = block_exclusive_scan(mine, wave_sum, tid, total);
        for (uint32_t b = b0; b < b1; ++b) {
            uint32_t lo, n;
            span(b, lo, n);
            for (uint32_t q = 0; q * kEmbRun < n; ++q)
                a.chunk_rec[at++] = make_uint2(lo + q * kEmbRun, b == a.n_buckets ? 0xFFFFFFFFu : b * a.bucket_rows);
        }
        if (tid == 0) {
            a.chunk_rec[total] = make_uint2(a.n_ids, 0xFFFFFFFFu);  // end marker
            *a.chunk_count = total;
        }
    }
#pragma unroll
    for (uint32_t r = 0; r < kEmbChunk / 1024; ++r) {
        const uint32_t i = tid + 1024 * r;
        if (i < a.n_ids) {
            const uint32_t at = first[slot[r]] + rank[r];
            a.keys[at] = key[r];
            a.pos[at] = i;
        }
    }
}

// Value of lane (l ^ kXor) for every lane l of the wavefront, without a trip through memory: quad
// permutes, row shifts and rotates inside a row of 16 lanes, and the two row / half swaps above that.
template <int kXor>
__device__ __forceinline__ uint32_t lane_xor(uint32_t x, uint32_t lane) {
    if (kXor == 1) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
    if (kXor == 2) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
    if (kXor == 4) {
        const uint32_t up = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x104, 0xF, 0xF, false);    // row_shl:4: from l + 4
        const uint32_t down = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x114, 0xF, 0xF, false);  // row_shr:4: from l - 4
        return (lane & 4u) ? down : up;
    }
    if (kXor == 8) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x128, 0xF, 0xF, false);  // row_ror:8
    if (kXor == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);  // {rows 0 and 2 doubled, rows 1 and 3 doubled}
        return (lane & 16u) ? r[0] : r[1];
    }
    const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);  // {lower half doubled, upper half doubled}
    return (lane & 32u) ? r[0] : r[1];
}

// One bitonic stage over the 64 lanes: ascending inside aligned blocks of 2 * kSize lanes ... with partner
// l ^ kStride; x is the same kind of word in every lane (larger = later).
template <int kSize, int kStride>
__device__ __forceinline__ uint32_t sort_stage(uint32_t x, uint32_t lane) {
    const uint32_t other = lane_xor<kStride>(x, lane);
    const bool keep_min = ((lane & kStride) == 0) == ((lane & kSize) == 0);
    return keep_min ? min(x, other) : max(x, other);
}

// The requests of a chunk (one per lane, `n` of them: row inside the bucket, < 2^26) in row order: returns
// (row << 6 | lane that held it) ascending over the lanes 0 .. n - 1.  Every lane must be active.  Only the
// stages that n needs are run; a chunk that arrives in order (the sorting kernel's) costs the same.
__device__ __forceinline__ uint32_t sort_chunk_rows(uint32_t row, uint32_t n, uint32_t lane) {
    uint32_t x = lane < n ? (row << 6) | lane : 0xFFFFFFFFu;
    if (n > 1) x = sort_stage<2, 1>(x, lane);
    if (n > 2) {
        x = sort_stage<4, 2>(x, lane);
        x = sort_stage<4, 1>(x, lane);
    }
    if (n > 4) {
        x = sort_stage<8, 4>(x, lane);
        x = sort_stage<8, 2>(x, lane);
        x = sort_stage<8, 1>(x, lane);
    }
    if (n > 8) {
        x = sort_stage<16, 8>(x, lane);
        x = sort_stage<16, 4>(x, lane);
        x = sort_stage<16, 2>(x, lane);
        x = sort_stage<16, 1>(x, lane);
    }
    if (n > 16) {
        x = sort_stage<32, 16>(x, lane);
        x = sort_stage<32, 8>(x, lane);
        x = sort_stage<32, 4>(x, lane);
        x = sort_stage<32, 2>(x, lane);
        x = sort_stage<32, 1>(x, lane);
    }
    if (n > 32) {
        x = sort_stage<64, 32>(x, lane);
        x = sort_stage<64, 16>(x, lane);
        x = sort_stage<64, 8>(x, lane);
        x = sort_stage<64, 4>(x, lane);
        x = sort_stage<64, 2>(x, lane);
        x = sort_stage<64, 1>(x, lane);
    }
    return x;
}

// One chunk of requests (all in one bucket = half tile of rows) for two neighbouring column tiles:
// lanes 0..31 the first tile's 32 streams of that half, lanes 32..63 the second tile's.  Walks the
// streams once, to the chunk's deepest row, and writes every requested row on the way as one
// 128-byte store.
// rec = the chunk's record {first request, its key}, hi = the first request of the next chunk.
// kStride = 0: no staging area of that kind; the item takes the guarded path.
template <uint32_t kStride>
__device__ __forceinline__ void embed_one_item(const EmbedArgs &a, uint2 rec, uint32_t hi, uint32_t pair,
                                               const uint2 *tab, uint8_t *stage, int lane) {
    const uint32_t lo = rec.x;
    if (lo >= hi || hi > a.n_ids) return;
    hi = min(hi, lo + kEmbRun);  // (chunks are cut at kEmbRun requests: one per lane)
    const uint32_t key0 = rec.y;
    const uint32_t b = key0 == 0xFFFFFFFFu ? a.n_buckets : min(key0 / a.bucket_rows, a.n_buckets - 1);
    const uint32_t c = lane % 32, side = lane / 32;
    const uint32_t tn = pair * 2 + side, col = tn * 32 + c;
    const bool col_ok = tn < a.tiles_n && col < a.N;
    if (b == a.n_buckets) {  // ids outside the table: zero rows
        for (uint32_t j = lo; j < hi; ++j)
            if (col_ok) a.out[(size_t)a.pos[j] * a.out_stride + col] = 0;
        return;
    }
    // bucket b = rows [b, b + 1) * bucket_rows: segment b % segs of half (b / segs) % 2 of k-tile b / (2 segs)
    const uint32_t half = a.th / 2, rows_b = a.bucket_rows, seg = b % a.segs, hsel = (b / a.segs) & 1,
                   tk = b / (2 * a.segs);
    const uint32_t tile_a = tk * a.tiles_n + pair * 2;
    const bool have_b = pair * 2 + 1 < a.tiles_n;
    const uint32_t tile_b = have_b ? tile_a + 1 : tile_a;
    uint64_t base_a = a.tile_offsets[tile_a], base_b = a.tile_offsets[tile_b];
    uint32_t depth_a = a.tile_max_lens[tile_a], depth_b = a.tile_max_lens[tile_b];
    if (base_a + (uint64_t)depth_a * 64 > a.stream_len) depth_a = 0;
    if (base_b + (uint64_t)depth_b * 64 > a.stream_len) depth_b = 0;
    const uint32_t tile = side ? tile_b : tile_a, depth = side ? depth_b : depth_a;
    const uint64_t base = side ? base_b : base_a;
    const uint32_t q = hsel * 32 + c;  // this lane's stream inside its tile
    // decoder state and row of the next unread byte at the first row of the bucket, and the row the
    // stream has reached at the bucket's end
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
    const uint32_t bucket_row0 = b * rows_b;
    const uint8_t *man = a.man_tiled + (size_t)tile * a.th * 32 + (size_t)(hsel * half + seg * rows_b) * 32 + c;
    // rows of the two bodies this item can touch (one window for both: neighbouring tiles lie alike)
    const int32_t w_lo = max(wave_min_i32(row_end) - 1, 0), w_hi = wave_max_i32(row);
    const uint32_t win_a = (uint32_t)max(min(w_hi + 1, (int32_t)depth_a) - w_lo, 0),
                   win_b = (uint32_t)max(min(w_hi + 1, (int32_t)depth_b) - w_lo, 0);
    const bool fast = kStride != 0 && __builtin_amdgcn_ballot_w64(!col_ok) == 0 && win_a >= 2 && win_b >= 2 &&
                      win_a < kStride && win_b < kStride && (uint32_t)(uintptr_t)tab == 0;
    // the chunk's requests in row order, one per lane: row inside the bucket and output position
    const uint32_t nb = hi - lo;
    const uint32_t raw_row = (uint32_t)lane < nb ? min(a.keys[lo + lane] - bucket_row0, rows_b - 1) : 0u;
    const uint32_t raw_pos = (uint32_t)lane < nb ? a.pos[lo + lane] : 0u;
    const uint32_t sorted = sort_chunk_rows(raw_row, nb, (uint32_t)lane);
    const uint32_t my_row = (uint32_t)lane < nb ? sorted >> 6 : 0u;
    const uint32_t my_pos = (uint32_t)__shfl((int)raw_pos, (int)(sorted & 63u), 64);
    if constexpr (kStride != 0) if (fast) {
        StageRegs body;
        const uint32_t deepest = max(win_a, win_b), my_depth = (lane & 4) ? win_b : win_a;
        const uint8_t *src_a = a.stream + base_a + (size_t)w_lo * 64, *src_b = a.stream + base_b + (size_t)w_lo * 64;
#pragma unroll
        for (int grp = 0; grp < stage_groups(kStride); ++grp)
            if ((uint32_t)grp * 128 < deepest) {
                stage_fetch_pair(body, src_a, win_a, src_b, win_b, hsel, grp * 128, lane);
                stage_commit<kStride>(body, stage, grp * 128, my_depth, lane);
            }
        FastLane st;
        st.init_at<kStride>(stage, row - w_lo + 1, lane, state);
        // The requests (read back from their lanes with readlane) are served in row order, their
        // sign|mantissa bytes fetched eight at a time, one group ahead of the decoding, so that no load
        // sits on the chain of decode steps.
        uint32_t done = 0, sym = 0;  // rows decoded so far, symbol of row done - 1
        {
            constexpr int kG = 8;
            uint32_t row_cur[kG] = {}, row_next[kG] = {};
            uint8_t man_cur[kG] = {}, man_next[kG] = {};
            auto fetch = [&](uint32_t first, uint32_t(&rows)[kG], uint8_t(&mans)[kG]) {
#pragma unroll
                for (int u = 0; u < kG; ++u) {
                    const uint32_t idx = min(first + u, nb - 1);  // wave uniform
                    rows[u] = min((uint32_t)__builtin_amdgcn_readlane((int)my_row, (int)idx), rows_b - 1);
                    mans[u] = man[(size_t)rows[u] * 32];
                }
            };
            fetch(0, row_cur, man_cur);
            for (uint32_t s0 = 0; s0 < nb; s0 += kG) {
                if (s0 + kG < nb) fetch(s0 + kG, row_next, man_next);
#pragma unroll
                for (int u = 0; u < kG; ++u)
                    if (s0 + u < nb) {
                        const uint32_t want = row_cur[u];
                        if (want + 1 > done) {  // wave uniform; sorted keys make the step count >= 1
                            sym = advance_asm(st, want + 1 - done) >> 24;
                            done = want + 1;
                        }
                        const uint32_t p = (uint32_t)__builtin_amdgcn_readlane((int)my_pos, (int)(s0 + u));
                        a.out[(size_t)p * a.out_stride + col] = (uint16_t)assemble_bf16(sym, man_cur[u]);
                    }
#pragma unroll
                for (int u = 0; u < kG; ++u) {
                    row_cur[u] = row_next[u];
                    man_cur[u] = man_next[u];
                }
            }
        }
        return;
    }
    GlobalBytes src;
    src.init(a.stream + base, (uint32_t)(row + 1), 64, q);
    uint32_t X = state << 3;
    const uint32_t last_row = (uint32_t)__builtin_amdgcn_readlane((int)my_row, (int)(nb - 1));  // deepest requested row
    uint32_t j = 0, want = (uint32_t)__builtin_amdgcn_readlane((int)my_row, 0);
    for (uint32_t i = 0; i <= last_row; ++i) {
        uint32_t sym = 0;
        if (col_ok) {
            sym = decode_symbol_scaled(X, tab) >> 24;
            src.renorm_scaled(X);
            src.renorm_scaled(X);
        }
        if (i == want) {  // wave uniform
            const uint16_t v = col_ok ? (uint16_t)assemble_bf16(sym, man[(size_t)i * 32]) : 0;
            do {
                const uint32_t p = (uint32_t)__builtin_amdgcn_readlane((int)my_pos, (int)j);
                if (col_ok) a.out[(size_t)p * a.out_stride + col] = v;
                ++j;
                want = j < nb ? (uint32_t)__builtin_amdgcn_readlane((int)my_row, (int)j) : 0xFFFFFFFFu;
            } while (want == i);
        }
    }
}

template <int kWaves, uint32_t kStride>
__device__ __forceinline__ void embed_wave_items(const EmbedArgs &a, const uint2 *tab, uint8_t *lds, int wave, int lane) {
    if (wave >= kWaves) return;
    uint8_t *stage = persist_stage<kWaves, kStride>(lds, wave);
    const uint32_t pairs = (a.tiles_n + 1) / 2;
    const uint64_t n_items = (uint64_t)min(*a.chunk_count, emb_max_chunks(a.n_ids, a.n_buckets)) * pairs;
    // An item's walk starts three dependent loads after its first one (chunk record -> tile offsets and
    // checkpoints -> body rows), and with checkpoints an item is short: the record of the next item is
    // fetched while this one runs.
    const uint64_t step = (uint64_t)kWaves * gridDim.x;
    auto record = [&](uint64_t item, uint2 &rec, uint32_t &hi) {
        const uint32_t chunk = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(item / pairs));
        rec = a.chunk_rec[chunk];
        hi = a.chunk_rec[chunk + 1].x;
    };
    uint64_t item = (uint64_t)wave * gridDim.x + blockIdx.x;
    uint2 rec = make_uint2(0u, 0u), next_rec = make_uint2(0u, 0u);
    uint32_t hi = 0, next_hi = 0;
    if (item < n_items) record(item, rec, hi);
    while (item < n_items) {
        if (item + step < n_items) record(item + step, next_rec, next_hi);
        embed_one_item<kStride>(a, rec, hi, (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(item % pairs)), tab,
                                stage, lane);
        rec = next_rec;
        hi = next_hi;
        item += step;
    }
}

// grid: at most one workgroup per CU, resident for the whole launch (fast_tile.h).  Work items are
// (chunk of requests, pair of column tiles), chunk-major, so the items of one requested row spread
// over as many workgroups as there are pairs.
__global__ __launch_bounds__(kPersistWaves *kWave) void embed_gather32_kernel(EmbedArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const uint32_t pairs = (a.tiles_n + 1) / 2;
    const uint64_t n_items = (uint64_t)min(*a.chunk_count, emb_max_chunks(a.n_ids, a.n_buckets)) * pairs;
    uint32_t deepest = 0;
    for (uint64_t item = (uint64_t)threadIdx.x * gridDim.x + blockIdx.x; item < n_items;
         item += (uint64_t)kPersistWaves * kWave * gridDim.x) {
        const uint2 rec = a.chunk_rec[item / pairs];
        const uint32_t pair = (uint32_t)(item % pairs), key0 = rec.y;
        if (rec.x >= a.n_ids) continue;
        if (key0 == 0xFFFFFFFFu) continue;  // the chunks of invalid ids touch no tile
        const uint32_t b = min(key0 / a.bucket_rows, a.n_buckets - 1);
        const uint32_t tile_a = (b / (2 * a.segs)) * a.tiles_n + pair * 2;
        deepest = max(deepest, a.tile_max_lens[tile_a]);
        if (pair * 2 + 1 < a.tiles_n) deepest = max(deepest, a.tile_max_lens[tile_a + 1]);
    }
    // a segment's window is about its share of the body plus the spread between the lanes; an item whose
    // window turns out larger than the class allows takes the guarded path
    if (a.segs > 1) deepest = deepest / a.segs + 40;
    // (this kernel measures a little faster on 10 wavefronts with 204-byte lane strides -- 51 dwords, odd, so
    // the lanes' bytes spread over the banks -- than on 11 with 186: the shallow class is not used)
    const uint32_t cls = persist_classify(lds, a.tables, a.slot_map, deepest);
    if (cls == 2u)
        embed_wave_items<8, kDepthDeep>(a, tab, lds, wave, lane);
    else if (cls == 3u)
        embed_wave_items<12, kDepthTiny>(a, tab, lds, wave, lane);
    else
        embed_wave_items<10, kDepthMedium>(a, tab, lds, wave, lane);
}

// ---- sixteen wavefronts per CU ------------------------------------------------------------------------
// With decoder checkpoints an item is short (a walk of at most bucket_rows steps) and what it costs is the
// chain of dependent loads in front of the walk: chunk record -> tile metadata, checkpoints and the chunk's
// requests -> body rows.  Sixteen wavefronts per CU (128 VGPRs, 7 KB of LDS each: stage_window_pair) walk
// their items with that chain taken apart: the record of the item three ahead, the metadata of the item two
// ahead and the window of the next item are on their way while the current item is decoded.  Items that do
// not qualify (ids outside the table, ragged columns, a window larger than the area) take embed_one_item's
// guarded path.
constexpr uint32_t kEmbSegBucketRows = 128;  // buckets up to this many rows go to this kernel

struct EmbRec {  // a chunk record as loaded (the same in every lane)
    uint32_t lo, key0, hi;
};
struct EmbRaw {  // what an item reads before its window is known
    uint32_t state, row, row_end;             // per lane, as stored (row: 0x7fffffff = from the body's last row)
    uint32_t off_a, depth_a, off_b, depth_b;  // the two tile bodies
    uint32_t key, pos;                        // this lane's request of the chunk
    uint32_t b, tile_a, tile_row0;            // the chunk's bucket (n_buckets: it touches no tile), its first tile,
                                              // the bucket's first row inside the tile
};
struct EmbItem {  // an item ready to be staged
    EmbRec rec;
    uint32_t pair;
    uint32_t nb, tile_a, tile_row0, bucket_row0;  // requests; first tile; first row of the bucket in its tile / in the table
    uint32_t state;
    int32_t row;
    uint32_t w_lo, rows, win_a, win_b;  // first body row of the window, rows in it (both bodies / each)
    uint32_t base_a, base_b;
    uint32_t my_row, my_pos;  // the chunk's requests in row order, one per lane
    bool fast;
};

__device__ __forceinline__ uint32_t uniform_u32(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

__device__ __forceinline__ void emb_rec_load(const EmbedArgs &a, uint32_t chunk, EmbRec &r) {
    const uint2 v = a.chunk_rec[chunk];
    r.lo = v.x;
    r.key0 = v.y;
    r.hi = a.chunk_rec[chunk + 1].x;
}

// The chunk's bucket, or n_buckets for a chunk that touches no tile (no requests, ids outside the table).
__device__ __forceinline__ uint32_t emb_bucket(const EmbedArgs &a, const EmbRec &r) {
    const uint32_t lo = uniform_u32(r.lo), hi = uniform_u32(r.hi), key0 = uniform_u32(r.key0);
    if (lo >= hi || hi > a.n_ids || key0 == 0xFFFFFFFFu) return a.n_buckets;
    return min(key0 / a.bucket_rows, a.n_buckets - 1);
}

__device__ __forceinline__ void emb_request(const EmbedArgs &a, const EmbRec &r, uint32_t pair, int lane, EmbRaw &m) {
    const uint32_t b = emb_bucket(a, r);
    m.state = m.row = m.row_end = m.off_a = m.depth_a = m.off_b = m.depth_b = m.key = m.pos = 0;
    m.b = b;
    m.tile_a = m.tile_row0 = 0;
    if (b == a.n_buckets) return;
    const uint32_t lo = uniform_u32(r.lo), nb = min(uniform_u32(r.hi) - lo, kEmbRun);
    const uint32_t bs = b / a.segs, seg = b - bs * a.segs, hsel = bs & 1, tk = bs / 2;
    const uint32_t side = lane / 32, c = lane % 32;
    const bool have_b = pair * 2 + 1 < a.tiles_n;
    const uint32_t tile_a = tk * a.tiles_n + pair * 2, tile_b = have_b ? tile_a + 1 : tile_a;
    m.tile_a = tile_a;
    m.tile_row0 = hsel * (a.th / 2) + seg * a.bucket_rows;
    m.off_a = a.tile_offsets[tile_a];
    m.depth_a = a.tile_max_lens[tile_a];
    m.off_b = a.tile_offsets[tile_b];
    m.depth_b = a.tile_max_lens[tile_b];
    const uint32_t tile = side ? tile_b : tile_a, q = hsel * 32 + c;
    const uint2 *ck = a.ckpt + ((size_t)tile * (a.segs - 1)) * 64 + q;
    if (seg == 0) {
        m.state = a.states[(size_t)tile * 64 + q];
        m.row = 0x7fffffffu;
    } else {
        const uint2 v = ck[(size_t)(seg - 1) * 64];
        m.state = v.x;
        m.row = v.y;
    }
    m.row_end = seg + 1 < a.segs ? ck[(size_t)seg * 64].y : 0xffffffffu;
    if ((uint32_t)lane < nb) {
        m.key = a.keys[lo + lane];
        m.pos = a.pos[lo + lane];
    }
}

// Same window and the same conditions as embed_one_item's, for the as-is staging area.
__device__ __forceinline__ void emb_resolve(const EmbedArgs &a, const EmbRec &r, uint32_t pair, int lane, const EmbRaw &m,
                                            EmbItem &it) {
    it.rec = r;
    it.pair = pair;
    it.fast = false;
    const uint32_t b = m.b;
    if (b == a.n_buckets) return;
    const uint32_t rows_b = a.bucket_rows;
    const uint32_t side = lane / 32, c = lane % 32, tn = pair * 2 + side, col = tn * 32 + c;
    it.nb = min(uniform_u32(r.hi) - uniform_u32(r.lo), kEmbRun);
    it.tile_a = m.tile_a;
    it.tile_row0 = m.tile_row0;
    it.bucket_row0 = b * rows_b;
    it.base_a = uniform_u32(m.off_a);
    it.base_b = uniform_u32(m.off_b);
    uint32_t depth_a = uniform_u32(m.depth_a), depth_b = uniform_u32(m.depth_b);
    if ((uint64_t)it.base_a + (uint64_t)depth_a * 64 > a.stream_len) depth_a = 0;
    if ((uint64_t)it.base_b + (uint64_t)depth_b * 64 > a.stream_len) depth_b = 0;
    const uint32_t depth = side ? depth_b : depth_a;
    it.state = m.state;
    it.row = min((int32_t)m.row, (int32_t)depth - 1);
    const int32_t row_end = min((int32_t)m.row_end, it.row);
    const bool col_ok = tn < a.tiles_n && col < a.N;
    const int32_t w_lo = max(wave_min_i32(row_end) - 1, 0), w_hi = wave_max_i32(it.row);
    it.w_lo = (uint32_t)w_lo;
    it.win_a = (uint32_t)max(min(w_hi + 1, (int32_t)depth_a) - w_lo, 0);
    it.win_b = (uint32_t)max(min(w_hi + 1, (int32_t)depth_b) - w_lo, 0);
    it.rows = max(it.win_a, it.win_b);
    it.fast = __builtin_amdgcn_ballot_w64(!col_ok) == 0 && it.win_a >= 2 && it.win_b >= 2 && it.rows <= kPairWinRows;
    // the chunk's requests in row order, one per lane: row inside the bucket and output position
    const uint32_t raw_row = (uint32_t)lane < it.nb ? min(m.key - it.bucket_row0, rows_b - 1) : 0u;
    const uint32_t sorted = sort_chunk_rows(raw_row, it.nb, (uint32_t)lane);
    it.my_row = (uint32_t)lane < it.nb ? sorted >> 6 : 0u;
    it.my_pos = (uint32_t)__shfl((int)m.pos, (int)(sorted & 63u), 64);
}

// Touches the cache lines of the item's two windows (a 128-byte line per lane and body); the values are not
// used, the caller keeps them alive until the current item has been decoded.
__device__ __forceinline__ void emb_touch(const EmbedArgs &a, const EmbItem &it, int lane, uint32_t &t, uint32_t &t2) {
    t = t2 = 0;
    if (!it.fast) return;
    if ((uint32_t)lane * 128 < it.win_a * 64)
        t = *reinterpret_cast<const uint32_t *>(a.stream + it.base_a + (size_t)it.w_lo * 64 + lane * 128);
    if ((uint32_t)lane * 128 < it.win_b * 64)
        t2 = *reinterpret_cast<const uint32_t *>(a.stream + it.base_b + (size_t)it.w_lo * 64 + lane * 128);
}

// A resolved, fast item: its window into the wavefront's area, then the walk to the chunk's deepest row; every
// requested row leaves as one 128-byte store (see embed_one_item).
__device__ __forceinline__ void emb_run(const EmbedArgs &a, const EmbItem &it, uint8_t *stage, int lane) {
    const uint32_t side = lane / 32, c = lane % 32, rows_b = a.bucket_rows, nb = it.nb;
    const uint32_t col = (it.pair * 2 + side) * 32 + c;
    const uint8_t *man = a.man_tiled + (size_t)(it.tile_a + side) * a.th * 32 + (size_t)it.tile_row0 * 32 + c;
    FastLane st;
    const int32_t rel = max(it.row - (int32_t)it.w_lo, -1);  // this lane's next byte, in rows of the window (-1: none left)
    st.X = it.state << 3;
    st.q = (uint32_t)(uintptr_t)stage + (uint32_t)(rel * 64 + lane);
    st.n1 = rel >= 0 ? stage[rel * 64 + lane] : 0;  // (a wavefront's LDS operations complete in order)
    const uint32_t my_row = it.my_row, my_pos = it.my_pos;
    uint32_t done = 0, sym = 0;  // rows decoded so far, symbol of row done - 1
    constexpr int kG = 8;
    uint32_t row_cur[kG] = {}, row_next[kG] = {};
    uint8_t man_cur[kG] = {}, man_next[kG] = {};
    auto fetch = [&](uint32_t first, uint32_t(&rows)[kG], uint8_t(&mans)[kG]) {
#pragma unroll
        for (int u = 0; u < kG; ++u) {
            const uint32_t idx = min(first + u, nb - 1);  // wave uniform
            rows[u] = min((uint32_t)__builtin_amdgcn_readlane((int)my_row, (int)idx), rows_b - 1);
            mans[u] = man[(size_t)rows[u] * 32];
        }
    };
    fetch(0, row_cur, man_cur);
    for (uint32_t s0 = 0; s0 < nb; s0 += kG) {
        if (s0 + kG < nb) fetch(s0 + kG, row_next, man_next);
#pragma unroll
        for (int u = 0; u < kG; ++u)
            if (s0 + u < nb) {
                const uint32_t want = row_cur[u];
                if (want + 1 > done) {  // wave uniform; requests in row order make the step count >= 1
                    sym = advance_asm(st, want + 1 - done, 64) >> 24;
                    done = want + 1;
                }
                const uint32_t p = (uint32_t)__builtin_amdgcn_readlane((int)my_pos, (int)(s0 + u));
                a.out[(size_t)p * a.out_stride + col] = (uint16_t)assemble_bf16(sym, man_cur[u]);
            }
#pragma unroll
        for (int u = 0; u < kG; ++u) {
            row_cur[u] = row_next[u];
            man_cur[u] = man_next[u];
        }
    }
}

// grid: at most one workgroup per CU; wavefront w of workgroup j takes the items j + (w + 16 i) * gridDim.x,
// chunk-major like embed_gather32_kernel.  The host launches it only when items number fewer than 2^31.
__global__ __launch_bounds__(kPairSegWaves *kWave) void embed_gather32_seg_kernel(EmbedArgs a, const uint2 *slot_table) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint2 *tab = reinterpret_cast<const uint2 *>(lds);
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t pairs = (a.tiles_n + 1) / 2;
    const uint32_t n_chunks = min(*a.chunk_count, emb_max_chunks(a.n_ids, a.n_buckets));
    uint8_t *stage = lds + kSlotTableBytes + (size_t)wave * kPairWinBytes;
    // (chunk, pair) of this wavefront's items, stepped without a division per item
    const uint32_t step = (uint32_t)kPairSegWaves * gridDim.x, step_q = step / pairs, step_r = step % pairs;
    const uint32_t first = (uint32_t)wave * gridDim.x + blockIdx.x;
    uint32_t ch2 = first / pairs, pr2 = first % pairs;  // the item whose record is asked for next
    auto advance = [&]() {
        ch2 += step_q;
        pr2 += step_r;
        if (pr2 >= pairs) {
            pr2 -= pairs;
            ++ch2;
        }
    };
    EmbRec r0 = {0, 0, 0}, r1 = r0, r2 = r0;
    uint32_t pr0 = 0, pr1 = 0;
    bool h0 = false, h1 = false, h2 = false;
    // the first three records, then the first item's metadata: on their way while the table arrives
    h0 = ch2 < n_chunks;
    if (h0) emb_rec_load(a, ch2, r0);
    pr0 = pr2;
    advance();
    h1 = h0 && ch2 < n_chunks;
    if (h1) emb_rec_load(a, ch2, r1);
    pr1 = pr2;
    advance();
    h2 = h1 && ch2 < n_chunks;
    if (h2) emb_rec_load(a, ch2, r2);
    EmbRaw raw;
    EmbItem nxt;
    nxt.fast = false;
    const bool tab_ok = (uint32_t)(uintptr_t)tab == 0;  // the hand-scheduled step reads the table at LDS address 0
    if (h0) emb_request(a, r0, pr0, lane, raw);
    if (slot_table) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(slot_table);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds);
        const u32x4 e0 = src[tid * 2], e1 = src[tid * 2 + 1];  // 1024 threads x 32 bytes = the 32 KB table
        dst[tid * 2] = e0;
        dst[tid * 2 + 1] = e1;
    } else {
        build_slot_table_x8(reinterpret_cast<uint2 *>(lds), a.tables, a.slot_map, tid, kPairSegWaves * kWave);
    }
    if (h0) {
        emb_resolve(a, r0, pr0, lane, raw, nxt);
        nxt.fast = nxt.fast && tab_ok;
        if (h1) emb_request(a, r1, pr1, lane, raw);
    }
    __syncthreads();
    while (h0) {
        const EmbItem cur = nxt;
        if (cur.fast)
            stage_window_pair(stage, a.stream + cur.base_a + (size_t)cur.w_lo * 64, cur.win_a,
                              a.stream + cur.base_b + (size_t)cur.w_lo * 64, cur.win_b, cur.tile_row0 >= a.th / 2 ? 1u : 0u,
                              cur.rows, lane);
        uint32_t touched = 0, touched2 = 0;
        h0 = h1;
        r0 = r1;
        pr0 = pr1;
        h1 = h2;
        r1 = r2;
        pr1 = pr2;
        if (h0) {
            emb_resolve(a, r0, pr0, lane, raw, nxt);
            nxt.fast = nxt.fast && tab_ok;
            emb_touch(a, nxt, lane, touched, touched2);
            if (h1) emb_request(a, r1, pr1, lane, raw);
        }
        if (h2) {
            advance();
            h2 = ch2 < n_chunks;
            if (h2) emb_rec_load(a, ch2, r2);
        }
        if (cur.fast)
            emb_run(a, cur, stage, lane);
        else
            embed_one_item<0>(a, make_uint2(uniform_u32(cur.rec.lo), uniform_u32(cur.rec.key0)), uniform_u32(cur.rec.hi),
                              cur.pair, tab, stage, lane);
        asm volatile("" ::"v"(touched), "v"(touched2));  // the touching loads end here
    }
}

// Any tile width, any tiled layout (TileLayout): one thread per (token, column), discarding the rows above
// the requested one exactly as the reference does (comp_inference/embedding_triton.py:239-257; one stream per column: :124-144).
template <int kLayout>
__global__ __launch_bounds__(256) void embed_generic_kernel(EmbedArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    const uint32_t col = blockIdx.y * 256 + threadIdx.x, m = blockIdx.x;
    if (col >= a.N) return;
    const int64_t id = a.ids[m];
    uint16_t *dst = a.out + (size_t)m * a.out_stride + col;
    if (id < 0 || id >= (int64_t)a.K) {
        *dst = 0;
        return;
    }
    const uint32_t tok = (uint32_t)id, tk = tok / a.th, rel = tok % a.th;
    const uint32_t tn = col / a.tw, c = col % a.tw, tile = tk * a.tiles_n + tn;
    constexpr bool kOne = kLayout != kBodyTwo;  // one stream per column over the whole tile height
    const uint32_t span = kOne ? a.th : a.th / 2, hsel = kOne ? 0 : rel / span, target = rel % span;
    uint32_t x, sym = 0;
    auto run = [&](auto &src) {
        for (uint32_t i = 0; i <= target; ++i) {
            sym = decode_symbol(x, tab) >> 24;
            src.renorm(x);
            src.renorm(x);
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
        const uint32_t spt = (kOne ? 1 : 2) * a.tw, q = hsel * a.tw + c;
        x = a.states[(size_t)tile * spt + q];
        uint64_t base = a.tile_offsets[tile];
        uint32_t depth = a.tile_max_lens[tile];
        if (base + (uint64_t)depth * spt > a.stream_len) depth = 0;
        GlobalBytes src;
        src.init(a.stream + base, depth, spt, q);
        run(src);
    }
    const uint32_t mb = a.man_tiled[(size_t)tile * a.th * a.tw + (size_t)rel * a.tw + c];
    *dst = (uint16_t)assemble_bf16(sym, mb);
}

}  // namespace ci

using namespace ci;

static uint32_t next_pow2(uint32_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

extern "C" size_t ci_fused_embedding_workspace_bytes_segmented(uint32_t n_ids, uint32_t K, uint32_t tile_height,
                                                               uint32_t segments) {
    if (segments == 0) segments = 1;
    if (tile_height < 2 || (tile_height / 2) % segments) return 0;
    const uint32_t chunk = n_ids < kEmbChunk ? n_ids : kEmbChunk;
    const uint32_t n_buckets = ceil_div(K, tile_height / 2 / segments);
    // sorted keys and positions, the chunk count, (8-byte aligned) one record per chunk and an end marker
    return (size_t)chunk * 8 + 4 + 8 + (size_t)(emb_max_chunks(chunk, n_buckets) + 1) * 8;
}

extern "C" size_t ci_fused_embedding_workspace_bytes(uint32_t n_ids, uint32_t K, uint32_t tile_height) {
    return ci_fused_embedding_workspace_bytes_segmented(n_ids, K, tile_height, 1);
}

static int embedding_impl(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream, uint64_t stream_len,
                          const uint32_t *d_states, const uint32_t *d_tables, const uint8_t *d_slot_map,
                          const uint32_t *d_meta0, const uint32_t *d_meta1, const uint8_t *d_man_tiled, uint32_t K,
                          uint32_t N, uint32_t th, uint32_t tw, uint16_t *d_out, uint32_t out_stride,
                          void *d_workspace, size_t workspace_bytes, int layout, hipStream_t s,
                          const void *d_checkpoints = nullptr, uint32_t segments = 1, const void *d_slot_table = nullptr) {
    const bool dense = layout != kBodyTwo;     // one stream per column: the one-thread-per-column kernel
    const bool exact = layout == kExactBytes;  // d_meta0 / d_meta1 are stream_offsets / stream_sizes
    if (n_ids == 0 || N == 0) return CI_OK;
    if (segments == 0) segments = 1;
    if (segments > 1) {
        if (dense || tw != 32 || (th & 1) || (th / 2) % segments)
            return fail(CI_ERR_ARG, "fused embedding: %u segments need 32-column tiles whose half height they divide", segments);
        if (!d_checkpoints || !aligned(d_checkpoints, 8))
            return fail(CI_ERR_ARG, "fused embedding: segments without (8-byte aligned) checkpoints");
    }
    if (!d_ids || !d_states || !d_tables || !d_slot_map || !d_meta0 || !d_meta1 || !d_man_tiled || !d_out)
        return fail(CI_ERR_ARG, "fused embedding: null pointer");
    if (stream_len && !d_stream) return fail(CI_ERR_ARG, "fused embedding: null stream");
    if (K == 0 || th == 0 || tw == 0 || (!dense && (th & 1))) return fail(CI_ERR_ARG, "fused embedding: bad shape");
    if (out_stride < N) return fail(CI_ERR_ARG, "fused embedding: row stride shorter than the row");
    if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "fused embedding: slot_map must be 4-byte aligned");

    EmbedArgs a;
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
    a.K = K;
    a.N = N;
    a.th = th;
    a.tw = tw;
    a.tiles_n = ceil_div(N, tw);
    a.out_stride = out_stride;
    a.ckpt = static_cast<const uint2 *>(d_checkpoints);
    a.segs = 1;
    a.bucket_rows = th / 2;

    const bool fast = !dense && tw == 32 && aligned(d_stream, 16);
    if (!fast) {
        a.ids = d_ids;
        a.n_ids = n_ids;
        a.out = d_out;
        a.n_buckets = 0;
        const dim3 grid(n_ids, ceil_div(N, 256)), block(256);
        if (layout == kExactBytes)
            hipLaunchKernelGGL(embed_generic_kernel<kExactBytes>, grid, block, 0, s, a);
        else if (layout == kBodyOne)
            hipLaunchKernelGGL(embed_generic_kernel<kBodyOne>, grid, block, 0, s, a);
        else
            hipLaunchKernelGGL(embed_generic_kernel<kBodyTwo>, grid, block, 0, s, a);
        CI_LAUNCH_CHECK("embed_generic_kernel");
        return CI_OK;
    }

    a.segs = segments;
    a.bucket_rows = th / 2 / segments;
    a.n_buckets = ceil_div(K, a.bucket_rows);
    const size_t need = ci_fused_embedding_workspace_bytes_segmented(n_ids, K, th, segments);
    if (!d_workspace || workspace_bytes < need)
        return fail(CI_ERR_CAPACITY, "fused embedding: workspace needs %zu bytes, got %zu", need, workspace_bytes);
    if (!aligned(d_workspace, 4)) return fail(CI_ERR_ARG, "fused embedding: workspace must be 4-byte aligned");
    const uint32_t chunk_cap = n_ids < kEmbChunk ? n_ids : kEmbChunk;
    a.keys = static_cast<uint32_t *>(d_workspace);
    a.pos = a.keys + chunk_cap;
    a.chunk_count = a.pos + chunk_cap;
    {   // the records behind the count, at the next 8-byte boundary
        uintptr_t at = reinterpret_cast<uintptr_t>(a.chunk_count + 1);
        a.chunk_rec = reinterpret_cast<uint2 *>((at + 7) & ~(uintptr_t)7);
    }
    CI_ALLOW_FULL_LDS(embed_gather32_kernel);
    CI_ALLOW_FULL_LDS(embed_gather32_seg_kernel);
    CI_ALLOW_FULL_LDS(embed_sort_kernel<true>);
    CI_ALLOW_FULL_LDS(embed_sort_kernel<false>);
    CI_ALLOW_FULL_LDS(embed_group_kernel);
    uint32_t cus = 0;
    if (int rc = cu_count(&cus)) return rc;
    // as many work items as chunks x pairs of column tiles; the chunk count is known on the device only
    // chunks run one after another on the stream and reuse the workspace
    for (uint32_t first = 0; first < n_ids; first += kEmbChunk) {
        a.ids = d_ids + first;
        a.n_ids = n_ids - first < kEmbChunk ? n_ids - first : kEmbChunk;
        a.out = d_out + (size_t)first * out_stride;
        a.n_pad = next_pow2(a.n_ids);
        // Counting slots: a bucket's rows, divided further (by powers of two) while there are no more slots
        // than ids -- then the chunks of a bucket that many ids fall into still cover ascending row ranges;
        // every slot costs time (0.7 ns: clearing, scanning), so few ids get few slots.
        uint32_t fine_rows = a.bucket_rows;
        while (fine_rows % 2 == 0 && ceil_div(K, fine_rows / 2) + 2 <= kGroupMaxSlots &&
               ceil_div(K, fine_rows / 2) <= a.n_ids)
            fine_rows /= 2;
        const uint32_t slots = ceil_div(K, fine_rows) + 2;
        if (slots <= kGroupMaxSlots) {
            hipLaunchKernelGGL(embed_group_kernel, dim3(1), dim3(1024), slots * 8 + 256, s, a, fine_rows);
            CI_LAUNCH_CHECK("embed_group_kernel");
        } else {  // more buckets than the counters hold: a full sort
            if (K < kEmbPackedInvalid)
                hipLaunchKernelGGL(embed_sort_kernel<true>, dim3(1), dim3(1024), a.n_pad * 8 + 4096, s, a);
            else
                hipLaunchKernelGGL(embed_sort_kernel<false>, dim3(1), dim3(1024), a.n_pad * 8 + 4096, s, a);
            CI_LAUNCH_CHECK("embed_sort_kernel");
        }
        const uint64_t most = (uint64_t)emb_max_chunks(a.n_ids, a.n_buckets) * ceil_div(a.tiles_n, 2u);
        const uint32_t gather_grid = (uint32_t)(most < (uint64_t)cus ? most : (uint64_t)cus);
        // Short buckets (decoder checkpoints) whose table the caller keeps beside the weight: sixteen wavefronts per
        // CU, every load of an item asked for ahead of it.
        if (segments > 1 && a.bucket_rows <= kEmbSegBucketRows && d_slot_table && aligned(d_slot_table, 16) &&
            most < (1ull << 31)) {
            hipLaunchKernelGGL(embed_gather32_seg_kernel, dim3(gather_grid), dim3(kPairSegWaves * kWave),
                               kSlotTableBytes + kPairSegWaves * kPairWinBytes, s, a,
                               static_cast<const uint2 *>(d_slot_table));
            CI_LAUNCH_CHECK("embed_gather32_seg_kernel");
            continue;
        }
        hipLaunchKernelGGL(embed_gather32_kernel, dim3(gather_grid), dim3(kPersistWaves * kWave), kLdsLimit, s, a);
        CI_LAUNCH_CHECK("embed_gather32_kernel");
    }
    return CI_OK;
}

extern "C" int ci_fused_embedding_ilp2(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                                       uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                                       const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                       const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled, uint32_t K,
                                       uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                                       uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                       ci_stream_t stream) {
    return embedding_impl(d_ids, n_ids, d_stream, stream_len, d_states, d_tables, d_slot_map, d_tile_offsets,
                          d_tile_max_lens, d_man_tiled, K, N, tile_height, tile_width, d_out, out_stride,
                          d_workspace, workspace_bytes, false, static_cast<hipStream_t>(stream));
}

extern "C" int ci_fused_embedding_ilp2_segmented(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                                                 uint64_t stream_len, const uint32_t *d_states,
                                                 const uint32_t *d_tables, const uint8_t *d_slot_map,
                                                 const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                                 const uint8_t *d_man_tiled, uint32_t K, uint32_t N,
                                                 uint32_t tile_height, uint32_t tile_width,
                                                 const void *d_checkpoints, uint32_t segments, uint16_t *d_out,
                                                 uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                                 ci_stream_t stream) {
    return embedding_impl(d_ids, n_ids, d_stream, stream_len, d_states, d_tables, d_slot_map, d_tile_offsets,
                          d_tile_max_lens, d_man_tiled, K, N, tile_height, tile_width, d_out, out_stride,
                          d_workspace, workspace_bytes, false, static_cast<hipStream_t>(stream), d_checkpoints,
                          segments);
}

extern "C" int ci_fused_embedding_tiled(const ci_tiled_weight *w, const int64_t *d_ids, uint32_t n_ids, uint16_t *d_out,
                                        uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                        ci_stream_t stream) {
    if (int rc = ci_tiled_weight_check(w)) return rc;
    if (!w->d_man_tiled) return fail(CI_ERR_ARG, "fused embedding: the weight has no sign|mantissa plane");
    const uint32_t segments = w->segments > 1 ? w->segments : 1;
    return embedding_impl(d_ids, n_ids, w->d_stream, w->stream_len, w->d_states, w->d_tables, w->d_slot_map,
                          w->d_tile_offsets, w->d_tile_max_lens, w->d_man_tiled, w->K, w->N, w->tile_height,
                          w->tile_width, d_out, out_stride, d_workspace, workspace_bytes, false,
                          static_cast<hipStream_t>(stream), segments > 1 ? w->d_checkpoints : nullptr, segments,
                          w->d_slot_table);
}

extern "C" int ci_fused_embedding_one(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                                      uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                                      const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                      const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled, uint32_t K,
                                      uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                                      uint32_t out_stride, ci_stream_t stream) {
    return embedding_impl(d_ids, n_ids, d_stream, stream_len, d_states, d_tables, d_slot_map, d_tile_offsets,
                          d_tile_max_lens, d_man_tiled, K, N, tile_height, tile_width, d_out, out_stride, nullptr,
                          0, kBodyOne, static_cast<hipStream_t>(stream));
}

extern "C" int ci_fused_embedding_dense(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                                        uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                                        const uint8_t *d_slot_map, const uint32_t *d_stream_offsets,
                                        const uint32_t *d_stream_sizes, const uint8_t *d_man_tiled, uint32_t K,
                                        uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                                        uint32_t out_stride, ci_stream_t stream) {
    return embedding_impl(d_ids, n_ids, d_stream, stream_len, d_states, d_tables, d_slot_map, d_stream_offsets,
                          d_stream_sizes, d_man_tiled, K, N, tile_height, tile_width, d_out, out_stride, nullptr,
                          0, true, static_cast<hipStream_t>(stream));
}
