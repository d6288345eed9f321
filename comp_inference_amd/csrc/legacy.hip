// Decoders of the two older stream layouts (gfx950): the flat layout and the dense tiled
// layout.  One thread per stream, the fused slot table in LDS, stream bytes read where they
// lie.  These layouts are kept for format compatibility; the tuned path is the tiled
// two-streams-per-column format in decode.hip.
#include "ci_common.h"
#include "rans_device.h"

namespace ci {

struct FlatArgs {
    const uint8_t *stream;
    uint64_t stream_len;
    const uint32_t *states;
    const uint32_t *sizes;
    const uint32_t *tables;
    const uint8_t *slot_map;
    uint32_t num_streams;
    uint32_t K, N;       // segmented variant
    uint64_t out_len;    // strided variant
    uint8_t *out;
};

// Bytes of stream g at [j * num_streams + g], read from j = size-1 downwards.
struct StridedBytes {
    const uint8_t *base;
    int64_t j;
    uint32_t stride;
    __device__ __forceinline__ void renorm(uint32_t &x) {
        if (x < kRansL && j >= 0) {
            x = (x << 8) | base[(size_t)j * stride];
            j -= 1;
        }
    }
};

// kSegmented: comp_inference/rans_triton.py:172-240 (stream g = 512-row segment g / N of
// column g % N).  !kSegmented: src/cuda/rans_kernels.cuh:626-708 (symbol i of stream g goes to
// out[g + i * streams], ceil(out_len / streams) symbols per stream).
template <bool kSegmented>
__global__ __launch_bounds__(256) void decode_flat_kernel(FlatArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    const uint32_t g = blockIdx.x * 256 + threadIdx.x;
    if (g >= a.num_streams) return;
    uint32_t size = a.sizes[g];
    // a size that would read past the stream is treated as empty
    if (size && (uint64_t)(size - 1) * a.num_streams + g >= a.stream_len) size = 0;
    StridedBytes src{a.stream + g, (int64_t)size - 1, a.num_streams};
    uint32_t x = a.states[g];
    if (kSegmented) {
        const uint32_t col = g % a.N, row0 = (g / a.N) * 512u;
        if (row0 >= a.K) return;
        const uint32_t n = min(512u, a.K - row0);
        for (uint32_t i = 0; i < n; ++i) {
            a.out[(size_t)(row0 + i) * a.N + col] = (uint8_t)(decode_symbol(x, tab) >> 24);
            src.renorm(x);
            src.renorm(x);
        }
    } else {
        const uint64_t per = (a.out_len + a.num_streams - 1) / a.num_streams;
        for (uint64_t i = 0; i < per; ++i) {
            const uint64_t o = g + i * a.num_streams;
            const uint32_t sym = decode_symbol(x, tab) >> 24;
            if (o < a.out_len) a.out[o] = (uint8_t)sym;  // the reference does not bound this write
            src.renorm(x);
            src.renorm(x);
        }
    }
}

struct DenseArgs {
    const uint8_t *stream;
    uint64_t stream_len;
    const uint32_t *states;
    const uint32_t *tables;
    const uint8_t *slot_map;
    const uint32_t *stream_offsets;
    const uint32_t *stream_sizes;
    uint32_t K, N, th, tw, tiles_n, num_streams;
    uint8_t *out_exp;
    const uint8_t *man_tiled;
    uint16_t *out_bf16;
};

// Stand-alone decode of the dense tiled layout (stream format:
// src/cuda/rans_kernels.cuh:7-74 + src/cuda/rans_ops.cu:165-176; byte order as read by
// comp_inference/linear_triton.py:1103-1108, :1147-1170).
template <bool kMerge>
__global__ __launch_bounds__(256) void decode_dense_kernel(DenseArgs a) {
    __shared__ uint2 tab[kProbScale];
    build_slot_table(tab, a.tables, a.slot_map, threadIdx.x, 256);
    __syncthreads();
    const uint32_t sid = blockIdx.x * 256 + threadIdx.x;
    if (sid >= a.num_streams) return;
    const uint32_t tile = sid / a.tw, c = sid % a.tw;
    const uint32_t tk = tile / a.tiles_n, tn = tile % a.tiles_n;
    const uint32_t col = tn * a.tw + c, row0 = tk * a.th;
    if (col >= a.N || row0 >= a.K) return;
    const uint32_t n = min(a.th, a.K - row0);
    const uint64_t off = a.stream_offsets[sid];
    uint32_t size = a.stream_sizes[sid];
    if (off + size > a.stream_len) size = 0;
    DenseBytes src;
    src.init(a.stream + off, size);
    uint32_t x = a.states[sid];
    const uint8_t *man = kMerge ? a.man_tiled + (size_t)tile * a.th * a.tw + c : nullptr;
    for (uint32_t i = 0; i < n; ++i) {
        const uint32_t sym = decode_symbol(x, tab) >> 24;
        src.renorm(x);
        src.renorm(x);
        const size_t o = (size_t)(row0 + i) * a.N + col;
        if (kMerge)
            a.out_bf16[o] = (uint16_t)assemble_bf16(sym, man[(size_t)i * a.tw]);
        else
            a.out_exp[o] = (uint8_t)sym;
    }
}

}  // namespace ci

using namespace ci;

static int check_flat(const void *stream, uint64_t stream_len, const void *states, const void *sizes,
                      uint32_t num_streams, const void *tables, const void *slot_map, const void *out) {
    if (num_streams == 0) return fail(CI_ERR_ARG, "flat decode: num_streams is 0");
    if (!states || !sizes || !tables || !slot_map || !out) return fail(CI_ERR_ARG, "flat decode: null pointer");
    if (stream_len && !stream) return fail(CI_ERR_ARG, "flat decode: null stream");
    if (!aligned(slot_map, 4)) return fail(CI_ERR_ARG, "flat decode: slot_map must be 4-byte aligned");
    return CI_OK;
}

extern "C" int ci_decode_flat_strided(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                      const uint32_t *d_sizes, uint32_t num_streams,
                                      const uint32_t *d_tables, const uint8_t *d_slot_map,
                                      uint64_t out_len, uint8_t *d_out, ci_stream_t stream) {
    if (out_len == 0) return CI_OK;
    int rc = check_flat(d_stream, stream_len, d_states, d_sizes, num_streams, d_tables, d_slot_map, d_out);
    if (rc) return rc;
    FlatArgs a{d_stream, stream_len, d_states, d_sizes, d_tables, d_slot_map, num_streams, 0, 0, out_len, d_out};
    hipLaunchKernelGGL(decode_flat_kernel<false>, dim3(ceil_div(num_streams, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    CI_LAUNCH_CHECK("decode_flat_kernel");
    return CI_OK;
}

extern "C" int ci_decode_flat_segmented(const uint8_t *d_stream, uint64_t stream_len,
                                        const uint32_t *d_states, const uint32_t *d_sizes,
                                        uint32_t num_streams, const uint32_t *d_tables,
                                        const uint8_t *d_slot_map, uint32_t K, uint32_t N, uint8_t *d_out,
                                        ci_stream_t stream) {
    if (K == 0 || N == 0) return CI_OK;
    int rc = check_flat(d_stream, stream_len, d_states, d_sizes, num_streams, d_tables, d_slot_map, d_out);
    if (rc) return rc;
    FlatArgs a{d_stream, stream_len, d_states, d_sizes, d_tables, d_slot_map, num_streams, K, N, 0, d_out};
    hipLaunchKernelGGL(decode_flat_kernel<true>, dim3(ceil_div(num_streams, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    CI_LAUNCH_CHECK("decode_flat_kernel");
    return CI_OK;
}

extern "C" int ci_decode_tiled_dense(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                     const uint32_t *d_tables, const uint8_t *d_slot_map,
                                     const uint32_t *d_stream_offsets, const uint32_t *d_stream_sizes,
                                     uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width,
                                     uint8_t *d_out_exp, const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                                     ci_stream_t stream) {
    if (K == 0 || N == 0) return CI_OK;
    if (!d_states || !d_tables || !d_slot_map || !d_stream_offsets || !d_stream_sizes)
        return fail(CI_ERR_ARG, "ci_decode_tiled_dense: null pointer");
    if (stream_len && !d_stream) return fail(CI_ERR_ARG, "ci_decode_tiled_dense: null stream");
    if (tile_height == 0 || tile_width == 0) return fail(CI_ERR_ARG, "ci_decode_tiled_dense: empty tile");
    if (!aligned(d_slot_map, 4)) return fail(CI_ERR_ARG, "ci_decode_tiled_dense: slot_map must be 4-byte aligned");
    const bool merge = d_man_tiled != nullptr;
    if (merge ? !d_out_bf16 : !d_out_exp) return fail(CI_ERR_ARG, "ci_decode_tiled_dense: null output");
    DenseArgs a;
    a.stream = d_stream;
    a.stream_len = stream_len;
    a.states = d_states;
    a.tables = d_tables;
    a.slot_map = d_slot_map;
    a.stream_offsets = d_stream_offsets;
    a.stream_sizes = d_stream_sizes;
    a.K = K;
    a.N = N;
    a.th = tile_height;
    a.tw = tile_width;
    a.tiles_n = ceil_div(N, tile_width);
    a.num_streams = ceil_div(K, tile_height) * a.tiles_n * tile_width;
    a.out_exp = d_out_exp;
    a.man_tiled = d_man_tiled;
    a.out_bf16 = d_out_bf16;
    const dim3 grid(ceil_div(a.num_streams, 256)), block(256);
    if (merge)
        hipLaunchKernelGGL(decode_dense_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream), a);
    else
        hipLaunchKernelGGL(decode_dense_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream), a);
    CI_LAUNCH_CHECK("decode_dense_kernel");
    return CI_OK;
}
