// Fused decompress + gather (embedding lookup) on gfx950.
//
// out[t, :] = table[ids[t], :] for a table stored as rANS-coded exponent plane + raw
// sign|mantissa plane; ids outside [0, K) give zero rows.  Replaces
// fused_rans_embedding_triton / fused_rans_embedding_kernel_ilp2
// (comp_inference/embedding_triton.py:170-330) and the dense-layout variant (:333-483).
//
// The reference starts one program per (token, column tile) and discards row % (th/2) decode
// steps in each.  Here the ids are sorted once (one workgroup, bitonic sort in LDS); a "bucket"
// is one half tile of rows, i.e. the row range of one stream.  Each wavefront owns one bucket
// of two neighbouring column tiles (32 + 32 lanes, all on the same half), walks the two half
// tiles once up to the deepest requested row and writes every requested row on the way as one
// 128-byte store.  Buckets nobody asked for exit before touching the stream.
#include "ci_common.h"
#include "rans_device.h"

namespace ci {

constexpr uint32_t kEmbChunk = 8192;  // ids sorted per pass (64 KB of LDS)
constexpr int kEmbWaves = 4;
constexpr uint32_t kEmbStageBytes = 14336;

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
    uint16_t *out;
    uint32_t out_stride;
    uint32_t *keys;          // workspace: sorted row ids (invalid = 0xFFFFFFFF, sorted last)
    uint32_t *pos;           // workspace: output row of each sorted id
    uint32_t *bucket_start;  // workspace: n_buckets + 2 entries (last real one = first invalid)
    uint32_t n_pad;          // n_ids rounded up to a power of two
    uint32_t stage_bytes;
};

// One workgroup: sort (id, position) by id, then mark where every bucket starts.
__global__ __launch_bounds__(1024) void embed_sort_kernel(EmbedArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t *key = reinterpret_cast<uint32_t *>(lds);
    uint32_t *val = key + a.n_pad;
    const uint32_t tid = threadIdx.x, half = a.th / 2;
    for (uint32_t i = tid; i < a.n_pad; i += 1024) {
        uint32_t k = 0xFFFFFFFFu;
        if (i < a.n_ids) {
            const int64_t id = a.ids[i];
            if (id >= 0 && id < (int64_t)a.K) k = (uint32_t)id;
        }
        key[i] = k;
        val[i] = i;
    }
    __syncthreads();
    for (uint32_t size = 2; size <= a.n_pad; size <<= 1)
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t t = tid; t < a.n_pad / 2; t += 1024) {
                const uint32_t lo = 2 * t - (t & (stride - 1)), hi = lo + stride;
                const bool up = (lo & size) == 0;
                const uint32_t ka = key[lo], kb = key[hi], va = val[lo], vb = val[hi];
                // ties are ordered by position so that the result does not depend on the network
                const bool gt = ka > kb || (ka == kb && va > vb);
                if (gt == up) {
                    key[lo] = kb;
                    key[hi] = ka;
                    val[lo] = vb;
                    val[hi] = va;
                }
            }
            __syncthreads();
        }
    const uint32_t nb = a.n_buckets + 1;  // bucket n_buckets collects the invalid ids
    for (uint32_t i = tid; i < a.n_ids; i += 1024) {
        a.keys[i] = key[i];
        a.pos[i] = val[i];
        const uint32_t b = key[i] == 0xFFFFFFFFu ? a.n_buckets : key[i] / half;
        const uint32_t pb = i == 0 ? 0 : (key[i - 1] == 0xFFFFFFFFu ? a.n_buckets : key[i - 1] / half);
        if (i == 0)
            for (uint32_t bb = 0; bb <= b; ++bb) a.bucket_start[bb] = 0;
        else
            for (uint32_t bb = pb + 1; bb <= b; ++bb) a.bucket_start[bb] = i;
    }
    __syncthreads();
    // buckets after the last occupied one, and the end marker
    if (tid == 0) {
        const uint32_t kl = a.n_ids ? key[a.n_ids - 1] : 0;
        const uint32_t bl = a.n_ids == 0 ? 0 : (kl == 0xFFFFFFFFu ? a.n_buckets : kl / half);
        for (uint32_t bb = (a.n_ids ? bl + 1 : 0); bb <= nb; ++bb) a.bucket_start[bb] = a.n_ids;
    }
}

// grid: (n_buckets + 1, ceil(tiles_n / (2 * kEmbWaves)))   block: kEmbWaves waves
__global__ __launch_bounds__(kEmbWaves *kWave) void embed_gather32_kernel(EmbedArgs a) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t b = blockIdx.x;
    const uint32_t lo = a.bucket_start[b], hi = a.bucket_start[b + 1];
    if (lo >= hi) return;  // uniform for the workgroup: nobody asked for this bucket
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const uint32_t c = lane % 32, side = lane / 32;
    const uint32_t tn = (blockIdx.y * kEmbWaves + wave) * 2 + side;
    const uint32_t col = tn * 32 + c;
    const bool col_ok = tn < a.tiles_n && col < a.N;

    if (b == a.n_buckets) {  // ids outside the table: zero rows
        for (uint32_t j = lo; j < hi; ++j)
            if (col_ok) a.out[(size_t)a.pos[j] * a.out_stride + col] = 0;
        return;
    }

    uint2 *tab = reinterpret_cast<uint2 *>(lds);
    // two tile bodies per wave, side by side
    uint8_t *stage = lds + kSlotTableBytes + ((size_t)wave * 2 + side) * a.stage_bytes;
    build_slot_table(tab, a.tables, a.slot_map, tid, kEmbWaves * kWave);

    const uint32_t half = a.th / 2, tk = b / 2, hsel = b & 1;
    const uint32_t tile = tk * a.tiles_n + (tn < a.tiles_n ? tn : 0);
    uint32_t depth = 0;
    uint64_t base = 0;
    if (tn < a.tiles_n) {
        base = a.tile_offsets[tile];
        depth = a.tile_max_lens[tile];
        if (base + (uint64_t)depth * 64 > a.stream_len) depth = 0;
    }
    // both halves of the wave must agree on the byte source; fall back together
    const bool fits = __builtin_amdgcn_ballot_w64(depth * 64u > a.stage_bytes) == 0;
    if (fits && tn < a.tiles_n) {
        // 32 lanes copy one body: 16 bytes per lane per pass
        for (uint32_t off = c * 16; off < depth * 64u; off += 32 * 16)
            *reinterpret_cast<u32x4 *>(stage + off) = *reinterpret_cast<const u32x4 *>(a.stream + base + off);
    }
    __syncthreads();

    const uint32_t q = hsel * 32 + c;  // this lane's stream inside its tile
    uint32_t x = tn < a.tiles_n ? a.states[(size_t)tile * 64 + q] : kRansL;
    const uint32_t bucket_row0 = b * half;
    const uint8_t *man = a.man_tiled + (size_t)tile * a.th * 32 + (size_t)hsel * half * 32 + c;
    const uint32_t last_row = a.keys[hi - 1] - bucket_row0;  // deepest requested row of the bucket

    auto walk = [&](auto &src) {
        uint32_t j = lo;
        uint32_t want = a.keys[j] - bucket_row0;
        for (uint32_t i = 0; i <= last_row; ++i) {
            const uint32_t sym = decode_symbol(x, tab) >> 24;
            src.renorm(x);
            src.renorm(x);
            if (i == want) {  // wave uniform
                const uint16_t v = (uint16_t)assemble_bf16(sym, man[(size_t)i * 32]);
                do {
                    if (col_ok) a.out[(size_t)a.pos[j] * a.out_stride + col] = v;
                    ++j;
                    want = j < hi ? a.keys[j] - bucket_row0 : 0xFFFFFFFFu;
                } while (want == i);
            }
        }
    };
    if (fits) {
        LdsBytes src;
        src.init(stage, depth, 64, q);
        walk(src);
    } else {
        GlobalBytes src;
        src.init(a.stream + base, depth, 64, q);
        walk(src);
    }
}

// Any tile width and the dense layout: one thread per (token, column), discarding the rows above
// the requested one exactly as the reference does (comp_inference/embedding_triton.py:239-257).
template <bool kDense>
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
    const uint32_t span = kDense ? a.th : a.th / 2, hsel = kDense ? 0 : rel / span, target = rel % span;
    uint32_t x, sym = 0;
    auto run = [&](auto &src) {
        for (uint32_t i = 0; i <= target; ++i) {
            sym = decode_symbol(x, tab) >> 24;
            src.renorm(x);
            src.renorm(x);
        }
    };
    if (kDense) {
        const uint32_t sid = tile * a.tw + c;
        x = a.states[sid];
        const uint64_t off = a.stream_offsets[sid];
        uint32_t size = a.stream_sizes[sid];
        if (off + size > a.stream_len) size = 0;
        DenseBytes src;
        src.init(a.stream + off, size);
        run(src);
    } else {
        const uint32_t spt = 2 * a.tw, q = hsel * a.tw + c;
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

extern "C" size_t ci_fused_embedding_workspace_bytes(uint32_t n_ids, uint32_t K, uint32_t tile_height) {
    if (tile_height < 2) return 0;
    const uint32_t chunk = n_ids < kEmbChunk ? n_ids : kEmbChunk;
    const uint32_t n_buckets = ceil_div(K, tile_height / 2);
    return (size_t)chunk * 8 + (size_t)(n_buckets + 3) * 4;
}

static int embedding_impl(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream, uint64_t stream_len,
                          const uint32_t *d_states, const uint32_t *d_tables, const uint8_t *d_slot_map,
                          const uint32_t *d_meta0, const uint32_t *d_meta1, const uint8_t *d_man_tiled, uint32_t K,
                          uint32_t N, uint32_t th, uint32_t tw, uint16_t *d_out, uint32_t out_stride,
                          void *d_workspace, size_t workspace_bytes, bool dense, hipStream_t s) {
    if (n_ids == 0 || N == 0) return CI_OK;
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
    a.tile_offsets = dense ? nullptr : d_meta0;
    a.tile_max_lens = dense ? nullptr : d_meta1;
    a.stream_offsets = dense ? d_meta0 : nullptr;
    a.stream_sizes = dense ? d_meta1 : nullptr;
    a.man_tiled = d_man_tiled;
    a.K = K;
    a.N = N;
    a.th = th;
    a.tw = tw;
    a.tiles_n = ceil_div(N, tw);
    a.out_stride = out_stride;
    a.stage_bytes = kEmbStageBytes;

    const bool fast = !dense && tw == 32 && aligned(d_stream, 16);
    if (!fast) {
        a.ids = d_ids;
        a.n_ids = n_ids;
        a.out = d_out;
        a.n_buckets = 0;
        const dim3 grid(n_ids, ceil_div(N, 256)), block(256);
        if (dense)
            hipLaunchKernelGGL(embed_generic_kernel<true>, grid, block, 0, s, a);
        else
            hipLaunchKernelGGL(embed_generic_kernel<false>, grid, block, 0, s, a);
        CI_LAUNCH_CHECK("embed_generic_kernel");
        return CI_OK;
    }

    a.n_buckets = ceil_div(K, th / 2);
    const size_t need = ci_fused_embedding_workspace_bytes(n_ids, K, th);
    if (!d_workspace || workspace_bytes < need)
        return fail(CI_ERR_CAPACITY, "fused embedding: workspace needs %zu bytes, got %zu", need, workspace_bytes);
    if (!aligned(d_workspace, 4)) return fail(CI_ERR_ARG, "fused embedding: workspace must be 4-byte aligned");
    const uint32_t chunk_cap = n_ids < kEmbChunk ? n_ids : kEmbChunk;
    a.keys = static_cast<uint32_t *>(d_workspace);
    a.pos = a.keys + chunk_cap;
    a.bucket_start = a.pos + chunk_cap;
    static bool attr_set = false;
    if (!attr_set) {
        CI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(embed_gather32_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
        CI_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(embed_sort_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit));
        attr_set = true;
    }
    const uint32_t gather_lds = kSlotTableBytes + kEmbWaves * 2 * a.stage_bytes;
    // chunks run one after another on the stream and reuse the workspace
    for (uint32_t first = 0; first < n_ids; first += kEmbChunk) {
        a.ids = d_ids + first;
        a.n_ids = n_ids - first < kEmbChunk ? n_ids - first : kEmbChunk;
        a.out = d_out + (size_t)first * out_stride;
        a.n_pad = next_pow2(a.n_ids);
        hipLaunchKernelGGL(embed_sort_kernel, dim3(1), dim3(1024), a.n_pad * 8, s, a);
        CI_LAUNCH_CHECK("embed_sort_kernel");
        hipLaunchKernelGGL(embed_gather32_kernel, dim3(a.n_buckets + 1, ceil_div(a.tiles_n, 2 * kEmbWaves)),
                           dim3(kEmbWaves * kWave), gather_lds, s, a);
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
