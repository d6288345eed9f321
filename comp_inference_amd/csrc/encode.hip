// rANS encoders (gfx950).  Encoding is the offline side of the format: one thread per stream
// walks its symbols bottom-up exactly as the reference's kernels do, writing the emitted bytes
// to a per-stream slice of a scratch buffer; the packing that the reference does in a
// single-threaded host loop runs here as small follow-up kernels on the same HIP stream.
//
// Three stream shapes share the one encode kernel:
//   kIlp2  two streams per (tile, column): rows [0,th/2) and [th/2,th)   (default format)
//   kDense one stream per (tile, column) over the full tile height       ("uncoalesced", and the first
//          tiled format, which packs these streams into tile bodies like the default one)
//   kFlat  stream gid = (512-row segment gid / N, column gid % N)         (legacy)
#include "ci_common.h"
#include "rans_device.h"

namespace ci {

enum Layout { kIlp2 = 0, kDense = 1, kFlat = 2 };

constexpr uint32_t kFlatSegment = 512;     // src/cuda/rans_kernels.cuh:421
constexpr uint32_t kCheckpointEvery = 128; // src/cuda/rans_kernels.cuh:5
constexpr size_t kHeaderBytes = 64;        // scratch header: [0] overflow flag, [1] max_len, [2..3] total

struct EncodeArgs {
    const uint8_t *symbols;
    const uint32_t *sym_info;  // 256 x (freq | cdf << 16), device copy at the scratch tail
    uint8_t *scratch;          // after the header
    uint32_t *header;
    uint32_t *states;
    uint32_t *sizes;
    uint64_t *checkpoints;     // flat only
    uint32_t K, N, th, tw, tiles_n, num_streams, capacity;
    int layout;
};

// src/cuda/rans_kernels.cuh:76-188 (kIlp2), :7-74 (kDense), :393-509 (kFlat)
__global__ __launch_bounds__(256) void encode_streams_kernel(EncodeArgs a) {
    __shared__ uint32_t info[256];
    info[threadIdx.x] = a.sym_info[threadIdx.x];
    __syncthreads();
    const uint32_t sid = blockIdx.x * 256 + threadIdx.x;
    if (sid >= a.num_streams) return;

    uint32_t col, r_lo, r_hi;  // this stream covers rows [r_lo, r_hi) of column col
    if (a.layout == kFlat) {
        col = sid % a.N;
        r_lo = (sid / a.N) * kFlatSegment;
        r_hi = r_lo + kFlatSegment;
    } else {
        const uint32_t spt = (a.layout == kIlp2 ? 2 : 1) * a.tw;
        const uint32_t tile = sid / spt, q = sid % spt;
        const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
        col = tn * a.tw + q % a.tw;
        if (a.layout == kIlp2) {
            r_lo = tk * a.th + (q / a.tw) * (a.th / 2);
            r_hi = r_lo + a.th / 2;
        } else {
            r_lo = tk * a.th;
            r_hi = r_lo + a.th;
        }
    }
    r_hi = min(r_hi, a.K);

    uint32_t x = kRansL, n_out = 0;
    uint8_t *dst = a.scratch + (size_t)sid * a.capacity;
    bool overflow = false;
    if (col < a.N && r_lo < r_hi) {
        const uint32_t n_sym = r_hi - r_lo;
        for (uint32_t i = 0; i < n_sym && !overflow; ++i) {
            if (a.layout == kFlat && i % kCheckpointEvery == 0)
                a.checkpoints[(size_t)(i / kCheckpointEvery) * a.num_streams + sid] =
                    (uint64_t)x | ((uint64_t)n_out << 32);
            const uint32_t row = r_hi - 1 - i;
            const uint32_t pk = info[a.symbols[(size_t)row * a.N + col]];
            const uint32_t f = pk & 0xFFFFu, c = pk >> 16;
            const uint32_t x_max = ((kRansL >> kProbBits) << 8) * f;
            while (x >= x_max) {
                if (n_out >= a.capacity) {
                    overflow = true;
                    break;
                }
                dst[n_out++] = (uint8_t)(x & 0xFFu);
                x >>= 8;
            }
            x = ((x / f) << kProbBits) + (x % f) + c;
        }
    }
    if (overflow) atomicOr(a.header, 1u);
    a.states[sid] = x;
    a.sizes[sid] = n_out;
}

// Longest stream of every tile (src/cuda/rans_ops.cu:340-346).  One thread per tile.
__global__ void tile_max_kernel(const uint32_t *sizes, uint32_t num_tiles, uint32_t spt,
                                uint32_t *tile_max_lens) {
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= num_tiles) return;
    uint32_t m = 0;
    for (uint32_t q = 0; q < spt; ++q) m = max(m, sizes[(size_t)t * spt + q]);
    tile_max_lens[t] = m;
}

// Exclusive scan of lens[i] * unit over n items by one workgroup; offsets are 32-bit as in
// the reference (src/cuda/rans_ops.cu:332), the 64-bit total goes to header[2..3].
__global__ __launch_bounds__(1024) void scan_offsets_kernel(const uint32_t *lens, uint32_t n,
                                                            uint32_t unit, uint32_t *offsets,
                                                            uint32_t *header) {
    __shared__ uint64_t part[1024];
    const uint32_t tid = threadIdx.x;
    const uint32_t per = (n + 1023) / 1024;
    const uint32_t lo = min(n, tid * per), hi = min(n, lo + per);
    uint64_t sum = 0;
    for (uint32_t i = lo; i < hi; ++i) sum += (uint64_t)lens[i] * unit;
    part[tid] = sum;
    __syncthreads();
    for (uint32_t d = 1; d < 1024; d <<= 1) {
        uint64_t v = tid >= d ? part[tid - d] : 0;
        __syncthreads();
        part[tid] += v;
        __syncthreads();
    }
    uint64_t run = part[tid] - sum;
    for (uint32_t i = lo; i < hi; ++i) {
        offsets[i] = (uint32_t)run;
        run += (uint64_t)lens[i] * unit;
    }
    if (tid == 1023) {
        header[2] = (uint32_t)part[1023];
        header[3] = (uint32_t)(part[1023] >> 32);
    }
}

__global__ __launch_bounds__(1024) void max_len_kernel(const uint32_t *sizes, uint32_t n,
                                                       uint32_t *header) {
    __shared__ uint32_t part[1024];
    uint32_t m = 0;
    for (uint32_t i = threadIdx.x; i < n; i += 1024) m = max(m, sizes[i]);
    part[threadIdx.x] = m;
    __syncthreads();
    for (uint32_t d = 512; d > 0; d >>= 1) {
        if (threadIdx.x < d) part[threadIdx.x] = max(part[threadIdx.x], part[threadIdx.x + d]);
        __syncthreads();
    }
    if (threadIdx.x == 0) header[1] = part[0];
}

// Tile body: max_len rows of spt bytes, each stream bottom-aligned under a zero prefix
// (src/cuda/rans_ops.cu:348-369).  One workgroup per tile, one byte per thread per pass.
__global__ __launch_bounds__(256) void pack_tiled_kernel(const uint8_t *scratch, const uint32_t *sizes,
                                                         const uint32_t *tile_offsets,
                                                         const uint32_t *tile_max_lens, uint32_t spt,
                                                         uint32_t capacity, uint8_t *stream,
                                                         uint64_t stream_len) {
    const uint32_t t = blockIdx.x;
    const uint32_t depth = tile_max_lens[t];
    const uint64_t base = tile_offsets[t];
    const uint32_t total = depth * spt;
    for (uint32_t e = threadIdx.x; e < total; e += 256) {
        const uint32_t r = e / spt, q = e % spt;
        const size_t sid = (size_t)t * spt + q;
        const uint32_t pad = depth - sizes[sid];
        if (base + e < stream_len) stream[base + e] = r < pad ? 0 : scratch[sid * capacity + (r - pad)];
    }
}

// Dense packing: stream sid's bytes copied to stream_offsets[sid] (src/cuda/rans_ops.cu:165-176).
__global__ __launch_bounds__(256) void pack_dense_kernel(const uint8_t *scratch, const uint32_t *sizes,
                                                         const uint32_t *stream_offsets,
                                                         uint32_t num_streams, uint32_t capacity,
                                                         uint8_t *stream, uint64_t stream_len) {
    const uint32_t sid = blockIdx.x * 256 + threadIdx.x;
    if (sid >= num_streams) return;
    const uint64_t off = stream_offsets[sid];
    const uint32_t n = sizes[sid];
    for (uint32_t j = 0; j < n; ++j)
        if (off + j < stream_len) stream[off + j] = scratch[(size_t)sid * capacity + j];
}

// Flat packing: byte j of stream g at [j * streams + g], max_len rows (src/cuda/rans_ops.cu:51-65).
__global__ __launch_bounds__(256) void pack_flat_kernel(const uint8_t *scratch, const uint32_t *sizes,
                                                        uint32_t num_streams, uint32_t capacity,
                                                        uint32_t max_len, uint8_t *stream) {
    const uint64_t e = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (uint64_t)max_len * num_streams) return;
    const uint32_t j = (uint32_t)(e / num_streams), g = (uint32_t)(e % num_streams);
    stream[e] = j < sizes[g] ? scratch[(size_t)g * capacity + j] : 0;
}

static uint32_t reference_capacity(uint64_t n_symbols, uint32_t n_streams) {
    // src/cuda/rans_host.cuh:470-471: (uint32_t)(syms_per_stream * 1.25) + 64
    const uint64_t per = (n_symbols + n_streams - 1) / n_streams;
    return (uint32_t)((double)per * 1.25) + 64u;
}

static size_t scratch_needed(uint32_t num_streams, uint32_t capacity) {
    return kHeaderBytes + 1024 + (size_t)num_streams * capacity;
}

// Shared front half of the three encoders: upload tables, encode, report overflow.
static int run_encode(const uint8_t *d_symbols, uint32_t K, uint32_t N, uint32_t th, uint32_t tw,
                      uint32_t tiles_n, uint32_t num_streams, uint32_t capacity, int layout,
                      const uint16_t *h_freqs, const uint16_t *h_cdf, uint8_t *d_scratch,
                      size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                      uint64_t *d_checkpoints, hipStream_t s) {
    if (!d_symbols || !h_freqs || !h_cdf || !d_scratch || !d_states || !d_sizes)
        return fail(CI_ERR_ARG, "encode: null pointer");
    if (scratch_bytes < scratch_needed(num_streams, capacity))
        return fail(CI_ERR_CAPACITY, "encode: scratch needs %zu bytes, got %zu",
                    scratch_needed(num_streams, capacity), scratch_bytes);
    uint32_t info[256];
    for (int i = 0; i < 256; ++i) {
        if (h_freqs[i] == 0) return fail(CI_ERR_ARG, "encode: symbol %d has frequency 0", i);
        info[i] = (uint32_t)h_freqs[i] | ((uint32_t)h_cdf[i] << 16);
    }
    uint32_t *header = reinterpret_cast<uint32_t *>(d_scratch);
    uint32_t *d_info = reinterpret_cast<uint32_t *>(d_scratch + kHeaderBytes);
    CI_HIP(hipMemsetAsync(header, 0, kHeaderBytes, s));
    CI_HIP(hipMemcpyAsync(d_info, info, sizeof info, hipMemcpyHostToDevice, s));
    // the table copy reads pageable host memory: finish it before `info` goes out of scope
    CI_HIP(hipStreamSynchronize(s));
    EncodeArgs a;
    a.symbols = d_symbols;
    a.sym_info = d_info;
    a.scratch = d_scratch + kHeaderBytes + 1024;
    a.header = header;
    a.states = d_states;
    a.sizes = d_sizes;
    a.checkpoints = d_checkpoints;
    a.K = K;
    a.N = N;
    a.th = th;
    a.tw = tw;
    a.tiles_n = tiles_n;
    a.num_streams = num_streams;
    a.capacity = capacity;
    a.layout = layout;
    hipLaunchKernelGGL(encode_streams_kernel, dim3(ceil_div(num_streams, 256)), dim3(256), 0, s, a);
    CI_LAUNCH_CHECK("encode_streams_kernel");
    return CI_OK;
}

static int read_header(const uint8_t *d_scratch, uint32_t h[4], hipStream_t s) {
    CI_HIP(hipMemcpyAsync(h, d_scratch, 16, hipMemcpyDeviceToHost, s));
    CI_HIP(hipStreamSynchronize(s));
    if (h[0] != 0) return fail(CI_ERR_ENCODE, "encode: a stream outgrew its capacity");
    return CI_OK;
}

}  // namespace ci

using namespace ci;

extern "C" int ci_tiling_init(ci_tiling *t, uint32_t K, uint32_t N, uint32_t tile_height,
                              uint32_t tile_width, int ilp2) {
    if (!t) return fail(CI_ERR_ARG, "ci_tiling_init: null");
    if (K == 0 || N == 0 || tile_height == 0 || tile_width == 0)
        return fail(CI_ERR_ARG, "ci_tiling_init: empty shape or tile");
    // src/cuda/rans_host.cuh:441-445
    if (ilp2 && tile_height % 16 != 0)
        return fail(CI_ERR_ARG, "Invalid tile height: must be a multiple of 16");
    if ((uint64_t)K * N >= (1ull << 32)) return fail(CI_ERR_ARG, "ci_tiling_init: K*N must be below 2^32");
    t->K = K;
    t->N = N;
    t->tile_height = tile_height;
    t->tile_width = tile_width;
    t->num_tiles_k = ceil_div(K, tile_height);
    t->num_tiles_n = ceil_div(N, tile_width);
    const uint64_t tiles = (uint64_t)t->num_tiles_k * t->num_tiles_n;
    t->streams_per_tile = (ilp2 ? 2u : 1u) * tile_width;
    if (tiles * t->streams_per_tile >= (1ull << 31)) return fail(CI_ERR_ARG, "ci_tiling_init: too many streams");
    t->num_tiles = (uint32_t)tiles;
    t->num_streams = t->num_tiles * t->streams_per_tile;
    t->capacity = reference_capacity((uint64_t)K * N, t->num_streams);
    return CI_OK;
}

extern "C" size_t ci_encode_scratch_bytes(uint32_t num_streams, uint32_t capacity) {
    return scratch_needed(num_streams, capacity);
}

// Encode, then the tile metadata of the two body layouts: depth of every tile and the scan of depth * spt.
static int encode_tiled_bodies(const char *who, int layout, const uint8_t *d_symbols, const ci_tiling *t,
                               const uint16_t *h_freqs, const uint16_t *h_cdf, uint8_t *d_scratch,
                               size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                               uint32_t *d_tile_offsets, uint32_t *d_tile_max_lens, uint64_t *h_stream_len,
                               hipStream_t s) {
    if (!t || !d_tile_offsets || !d_tile_max_lens || !h_stream_len) return fail(CI_ERR_ARG, "%s: null pointer", who);
    if (t->streams_per_tile != (layout == kIlp2 ? 2u : 1u) * t->tile_width)
        return fail(CI_ERR_ARG, "%s: tiling was not initialised for %s per column", who,
                    layout == kIlp2 ? "two streams" : "one stream");
    int rc = run_encode(d_symbols, t->K, t->N, t->tile_height, t->tile_width, t->num_tiles_n,
                        t->num_streams, t->capacity, layout, h_freqs, h_cdf, d_scratch, scratch_bytes,
                        d_states, d_sizes, nullptr, s);
    if (rc) return rc;
    uint32_t *header = reinterpret_cast<uint32_t *>(d_scratch);
    hipLaunchKernelGGL(tile_max_kernel, dim3(ceil_div(t->num_tiles, 256)), dim3(256), 0, s, d_sizes,
                       t->num_tiles, t->streams_per_tile, d_tile_max_lens);
    CI_LAUNCH_CHECK("tile_max_kernel");
    hipLaunchKernelGGL(scan_offsets_kernel, dim3(1), dim3(1024), 0, s, d_tile_max_lens, t->num_tiles,
                       t->streams_per_tile, d_tile_offsets, header);
    CI_LAUNCH_CHECK("scan_offsets_kernel");
    uint32_t h[4];
    rc = read_header(d_scratch, h, s);
    if (rc) return rc;
    *h_stream_len = (uint64_t)h[2] | ((uint64_t)h[3] << 32);
    return CI_OK;
}

static int pack_tiled_bodies(const char *who, const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                             const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens, uint8_t *d_stream,
                             uint64_t stream_len, hipStream_t s) {
    if (!d_scratch || !t || !d_sizes || !d_tile_offsets || !d_tile_max_lens) return fail(CI_ERR_ARG, "%s: null pointer", who);
    if (stream_len == 0) return CI_OK;
    if (!d_stream) return fail(CI_ERR_ARG, "%s: null stream buffer", who);
    hipLaunchKernelGGL(pack_tiled_kernel, dim3(t->num_tiles), dim3(256), 0, s,
                       d_scratch + kHeaderBytes + 1024, d_sizes, d_tile_offsets, d_tile_max_lens,
                       t->streams_per_tile, t->capacity, d_stream, stream_len);
    CI_LAUNCH_CHECK("pack_tiled_kernel");
    return CI_OK;
}

extern "C" int ci_encode_tiled_ilp2(const uint8_t *d_symbols, const ci_tiling *t,
                                    const uint16_t *h_freqs, const uint16_t *h_cdf, uint8_t *d_scratch,
                                    size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                                    uint32_t *d_tile_offsets, uint32_t *d_tile_max_lens,
                                    uint64_t *h_stream_len, ci_stream_t stream) {
    return encode_tiled_bodies("ci_encode_tiled_ilp2", kIlp2, d_symbols, t, h_freqs, h_cdf, d_scratch, scratch_bytes,
                               d_states, d_sizes, d_tile_offsets, d_tile_max_lens, h_stream_len,
                               static_cast<hipStream_t>(stream));
}

extern "C" int ci_pack_tiled_ilp2(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                                  const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                  uint8_t *d_stream, uint64_t stream_len, ci_stream_t stream) {
    if (t && t->streams_per_tile != 2 * t->tile_width)
        return fail(CI_ERR_ARG, "ci_pack_tiled_ilp2: tiling was not initialised for two streams per column");
    return pack_tiled_bodies("ci_pack_tiled_ilp2", d_scratch, t, d_sizes, d_tile_offsets, d_tile_max_lens, d_stream,
                             stream_len, static_cast<hipStream_t>(stream));
}

// src/cuda/rans_kernels.cuh:316-391 + src/cuda/rans_ops.cu:412-600
extern "C" int ci_encode_tiled_one(const uint8_t *d_symbols, const ci_tiling *t,
                                   const uint16_t *h_freqs, const uint16_t *h_cdf, uint8_t *d_scratch,
                                   size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                                   uint32_t *d_tile_offsets, uint32_t *d_tile_max_lens,
                                   uint64_t *h_stream_len, ci_stream_t stream) {
    return encode_tiled_bodies("ci_encode_tiled_one", kDense, d_symbols, t, h_freqs, h_cdf, d_scratch, scratch_bytes,
                               d_states, d_sizes, d_tile_offsets, d_tile_max_lens, h_stream_len,
                               static_cast<hipStream_t>(stream));
}

extern "C" int ci_pack_tiled_one(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                                 const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                 uint8_t *d_stream, uint64_t stream_len, ci_stream_t stream) {
    if (t && t->streams_per_tile != t->tile_width)
        return fail(CI_ERR_ARG, "ci_pack_tiled_one: tiling was not initialised for one stream per column");
    return pack_tiled_bodies("ci_pack_tiled_one", d_scratch, t, d_sizes, d_tile_offsets, d_tile_max_lens, d_stream,
                             stream_len, static_cast<hipStream_t>(stream));
}

extern "C" int ci_encode_tiled_dense(const uint8_t *d_symbols, const ci_tiling *t,
                                     const uint16_t *h_freqs, const uint16_t *h_cdf, uint8_t *d_scratch,
                                     size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                                     uint32_t *d_stream_offsets, uint64_t *h_stream_len,
                                     ci_stream_t stream) {
    if (!t || !d_stream_offsets || !h_stream_len) return fail(CI_ERR_ARG, "ci_encode_tiled_dense: null pointer");
    if (t->streams_per_tile != t->tile_width)
        return fail(CI_ERR_ARG, "ci_encode_tiled_dense: tiling was not initialised for one stream per column");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = run_encode(d_symbols, t->K, t->N, t->tile_height, t->tile_width, t->num_tiles_n,
                        t->num_streams, t->capacity, kDense, h_freqs, h_cdf, d_scratch, scratch_bytes,
                        d_states, d_sizes, nullptr, s);
    if (rc) return rc;
    uint32_t *header = reinterpret_cast<uint32_t *>(d_scratch);
    hipLaunchKernelGGL(scan_offsets_kernel, dim3(1), dim3(1024), 0, s, d_sizes, t->num_streams, 1u,
                       d_stream_offsets, header);
    CI_LAUNCH_CHECK("scan_offsets_kernel");
    uint32_t h[4];
    rc = read_header(d_scratch, h, s);
    if (rc) return rc;
    *h_stream_len = (uint64_t)h[2] | ((uint64_t)h[3] << 32);
    return CI_OK;
}

extern "C" int ci_pack_tiled_dense(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                                   const uint32_t *d_stream_offsets, uint8_t *d_stream,
                                   uint64_t stream_len, ci_stream_t stream) {
    if (!d_scratch || !t || !d_sizes || !d_stream_offsets) return fail(CI_ERR_ARG, "ci_pack_tiled_dense: null pointer");
    if (stream_len == 0) return CI_OK;
    if (!d_stream) return fail(CI_ERR_ARG, "ci_pack_tiled_dense: null stream buffer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(pack_dense_kernel, dim3(ceil_div(t->num_streams, 256)), dim3(256), 0, s,
                       d_scratch + kHeaderBytes + 1024, d_sizes, d_stream_offsets, t->num_streams,
                       t->capacity, d_stream, stream_len);
    CI_LAUNCH_CHECK("pack_dense_kernel");
    return CI_OK;
}

extern "C" int ci_flat_geometry(uint32_t K, uint32_t N, uint32_t min_block_size, uint32_t *num_streams,
                                uint32_t *capacity) {
    if (K == 0 || N == 0 || min_block_size == 0 || !num_streams || !capacity)
        return fail(CI_ERR_ARG, "ci_flat_geometry: empty shape, zero block size or null pointer");
    // src/cuda/rans_host.cuh:176-182
    const uint64_t streams = (uint64_t)ceil_div(K, min_block_size) * N;
    if (streams >= (1ull << 31) || (uint64_t)K * N >= (1ull << 32))
        return fail(CI_ERR_ARG, "ci_flat_geometry: shape too large");
    *num_streams = (uint32_t)streams;
    *capacity = reference_capacity((uint64_t)K * N, (uint32_t)streams);
    return CI_OK;
}

extern "C" int ci_encode_flat(const uint8_t *d_symbols, uint32_t K, uint32_t N, uint32_t num_streams,
                              uint32_t capacity, const uint16_t *h_freqs, const uint16_t *h_cdf,
                              uint8_t *d_scratch, size_t scratch_bytes, uint32_t *d_states,
                              uint32_t *d_sizes, uint64_t *d_checkpoints, uint32_t *h_max_len,
                              ci_stream_t stream) {
    if (!d_checkpoints || !h_max_len) return fail(CI_ERR_ARG, "ci_encode_flat: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    CI_HIP(hipMemsetAsync(d_checkpoints, 0, (size_t)num_streams * kCheckpointEvery * sizeof(uint64_t), s));
    int rc = run_encode(d_symbols, K, N, 0, 0, 0, num_streams, capacity, kFlat, h_freqs, h_cdf, d_scratch,
                        scratch_bytes, d_states, d_sizes, d_checkpoints, s);
    if (rc) return rc;
    hipLaunchKernelGGL(max_len_kernel, dim3(1), dim3(1024), 0, s, d_sizes, num_streams,
                       reinterpret_cast<uint32_t *>(d_scratch));
    CI_LAUNCH_CHECK("max_len_kernel");
    uint32_t h[4];
    rc = read_header(d_scratch, h, s);
    if (rc) return rc;
    *h_max_len = h[1];
    return CI_OK;
}

extern "C" int ci_pack_flat(const uint8_t *d_scratch, uint32_t num_streams, uint32_t capacity,
                            const uint32_t *d_sizes, uint32_t max_len, uint8_t *d_stream,
                            ci_stream_t stream) {
    if (!d_scratch || !d_sizes) return fail(CI_ERR_ARG, "ci_pack_flat: null pointer");
    const uint64_t total = (uint64_t)max_len * num_streams;
    if (total == 0) return CI_OK;
    if (!d_stream) return fail(CI_ERR_ARG, "ci_pack_flat: null stream buffer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(pack_flat_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s,
                       d_scratch + kHeaderBytes + 1024, d_sizes, num_streams, capacity, max_len, d_stream);
    CI_LAUNCH_CHECK("pack_flat_kernel");
    return CI_OK;
}

extern "C" int ci_build_tables(const uint16_t *h_freqs, const uint16_t *h_cdf, uint32_t *h_tables,
                               uint8_t *h_slot_map) {
    if (!h_freqs || !h_cdf || !h_tables || !h_slot_map) return fail(CI_ERR_ARG, "ci_build_tables: null pointer");
    for (int i = 0; i < 256; ++i) {
        h_tables[i] = (uint32_t)h_freqs[i] | ((uint32_t)h_cdf[i] << 16);
        for (uint32_t j = 0; j < h_freqs[i]; ++j) {
            const uint32_t slot = (uint32_t)h_cdf[i] + j;
            if (slot >= kProbScale) return fail(CI_ERR_ARG, "ci_build_tables: cdf + freq exceeds 4096 at symbol %d", i);
            h_slot_map[slot] = (uint8_t)i;
        }
    }
    return CI_OK;
}
