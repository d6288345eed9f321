/*
 * comp_inference_hip.h -- C ABI of libcomp_inference_hip.so (MI355X / gfx950).
 *
 * This library stands where the reference's pybind11/CUDA extension `comp_inference.ccore`
 * (src/python_bindings.cpp:59-472) and its Triton kernels stand: rANS coding of the bf16
 * exponent plane and the fused decode kernels.  Every entry point takes plain pointers and
 * sizes; "d_" arguments are device pointers, "h_" arguments are host pointers.  Kernels are
 * enqueued on the given hipStream_t and, unless a function says otherwise, the call does not
 * wait for them (the reference's ops run on the current torch stream without a sync,
 * src/cuda/rans_host.cuh:823-834).
 *
 * Return value: 0 on success, a CI_ERR_* code otherwise; ci_last_error() then holds a
 * message (thread local).  The reference reports the same conditions as C++ exceptions that
 * pybind11 turns into RuntimeError (src/cuda/rans_host.cuh:12-20, :441-445, :462-467).
 *
 * Coder parameters are the reference's RansConfig8 (src/cuda/rans_host.cuh:22-24): 8-bit
 * symbols, 12-bit probabilities, byte I/O, 32-bit state with lower bound 2^16.
 */
#ifndef COMP_INFERENCE_HIP_H
#define COMP_INFERENCE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CI_OK 0
#define CI_ERR_ARG 1      /* bad shape, size, alignment or null pointer            */
#define CI_ERR_HIP 2      /* a HIP runtime call or kernel launch failed            */
#define CI_ERR_CAPACITY 3 /* a buffer handed in by the caller is too small         */
#define CI_ERR_DEVICE 4   /* current device is not gfx950                          */
#define CI_ERR_ENCODE 5   /* a stream outgrew the per-stream capacity              */

typedef void *ci_stream_t; /* a hipStream_t; NULL = the null stream */

/* Message of the last failing call on this thread ("" if none). */
const char *ci_last_error(void);

/* ABI version of this header (bumped when a signature changes). */
int ci_abi_version(void);

/* CI_OK if the current HIP device is a gfx950; CI_ERR_DEVICE otherwise.  There is no
 * fallback path: on any other device the library refuses to run. */
int ci_check_device(void);

/* ---------------------------------------------------------------------------------------
 * Geometry of a tiled encoding (src/cuda/rans_host.cuh:447-471).  ilp2 != 0: two streams
 * per column per tile (the default format); ilp2 == 0: one stream per column per tile (the
 * dense / "uncoalesced" format).  capacity = bytes reserved per stream in the scratch buffer.
 * ------------------------------------------------------------------------------------- */
typedef struct ci_tiling {
    uint32_t K, N, tile_height, tile_width;
    uint32_t num_tiles_k, num_tiles_n, num_tiles;
    uint32_t streams_per_tile, num_streams;
    uint32_t capacity;
} ci_tiling;

int ci_tiling_init(ci_tiling *t, uint32_t K, uint32_t N, uint32_t tile_height,
                   uint32_t tile_width, int ilp2);

/* ---------------------------------------------------------------------------------------
 * Encoder, default format.  Replaces RansManager::compress_tiled_ilp2
 * (src/cuda/rans_ops.cu:205-410) = kernel rans_compress_kernel_tiled_ilp2
 * (src/cuda/rans_kernels.cuh:76-188) + the host interleave loop (src/cuda/rans_ops.cu:328-375),
 * which here runs on the GPU as a second kernel.
 *
 * Step 1, ci_encode_tiled_ilp2: encodes d_symbols (u8 [K,N] row major) into d_scratch
 * (num_streams * capacity bytes), fills d_states / d_sizes (num_streams each) and
 * d_tile_offsets / d_tile_max_lens (num_tiles each), waits for the stream and returns the
 * packed length in *h_stream_len.  CI_ERR_ENCODE if any stream outgrew `capacity` (the
 * reference loses that flag in a by-value kernel argument, src/cuda/rans_kernels.cuh:144-146).
 * Step 2, ci_pack_tiled_ilp2: writes the packed stream (exactly *h_stream_len bytes) into
 * d_stream.  Streams of columns >= N get state 2^16 and size 0.
 * ------------------------------------------------------------------------------------- */
int ci_encode_tiled_ilp2(const uint8_t *d_symbols, const ci_tiling *t, const uint16_t *h_freqs,
                         const uint16_t *h_cdf, uint8_t *d_scratch, size_t scratch_bytes,
                         uint32_t *d_states, uint32_t *d_sizes, uint32_t *d_tile_offsets,
                         uint32_t *d_tile_max_lens, uint64_t *h_stream_len, ci_stream_t stream);

int ci_pack_tiled_ilp2(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                       const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                       uint8_t *d_stream, uint64_t stream_len, ci_stream_t stream);

/* Host-side decoder tables (src/cuda/rans_host.cuh:476-488): tables[s] = freq | cdf << 16,
 * slot_map[cdf[s] + j] = s.  h_tables: 256 entries, h_slot_map: 4096 entries. */
int ci_build_tables(const uint16_t *h_freqs, const uint16_t *h_cdf, uint32_t *h_tables,
                    uint8_t *h_slot_map);

/* ---------------------------------------------------------------------------------------
 * Stand-alone decoder, default format.  Replaces rans_decomp_triton_tiled /
 * rans_decompress_tiled_kernel_triton_ilp2 (comp_inference/rans_triton.py:34-168).
 * Output: the exponent plane, u8 [K,N] row major.
 * d_man_tiled != NULL additionally merges the tile-interleaved sign|mantissa plane
 * (comp_inference/comp_inference.py:35-64) and writes bf16 bit patterns to d_out_bf16
 * (the reference does this merge as separate torch ops, comp_inference/comp_inference.py:694-708).
 * ------------------------------------------------------------------------------------- */
int ci_decode_tiled_ilp2(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                         const uint32_t *d_tables, const uint8_t *d_slot_map,
                         const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                         uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width,
                         uint8_t *d_out_exp, const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                         ci_stream_t stream);

/* Bytes of scratch the encoders need for `num_streams` streams of `capacity` bytes (a small
 * header for flags and totals precedes the per-stream slices). */
size_t ci_encode_scratch_bytes(uint32_t num_streams, uint32_t capacity);

/* ---------------------------------------------------------------------------------------
 * Encoder, dense ("uncoalesced") format: one stream per (tile, column) over the full tile
 * height, streams concatenated byte-exact.  Replaces RansManager::compress_tiled_uncoalesced
 * (src/cuda/rans_ops.cu:74-203) = kernel rans_compress_kernel_tiled_uncoalesced
 * (src/cuda/rans_kernels.cuh:7-74) + the host packing loop (src/cuda/rans_ops.cu:165-176).
 * Same two-step protocol as the default format; d_stream_offsets has num_streams entries.
 * The tiling must come from ci_tiling_init(..., ilp2 = 0).
 * ------------------------------------------------------------------------------------- */
int ci_encode_tiled_dense(const uint8_t *d_symbols, const ci_tiling *t, const uint16_t *h_freqs,
                          const uint16_t *h_cdf, uint8_t *d_scratch, size_t scratch_bytes,
                          uint32_t *d_states, uint32_t *d_sizes, uint32_t *d_stream_offsets,
                          uint64_t *h_stream_len, ci_stream_t stream);

int ci_pack_tiled_dense(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                        const uint32_t *d_stream_offsets, uint8_t *d_stream, uint64_t stream_len,
                        ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * The first tiled format: one stream per (tile, column) over the full tile height, packed into
 * tile bodies like the default format -- tile_max_lens[t] rows of tile_width bytes, stream q in
 * byte column q, bottom-aligned under a zero prefix, tile_offsets = scan of depth * tile_width.
 * ci_encode_tiled_one / ci_pack_tiled_one replace RansManager::compress_tiled
 * (src/cuda/rans_ops.cu:412-600) = kernel rans_compress_kernel_tiled
 * (src/cuda/rans_kernels.cuh:316-391) + the host packing loop (src/cuda/rans_ops.cu:522-566);
 * same two-step protocol and arguments as ci_encode_tiled_ilp2 / ci_pack_tiled_ilp2, with a tiling
 * from ci_tiling_init(..., ilp2 = 0).  The reference's Python module does not bind this encoder
 * (src/python_bindings.cpp:302-347 binds the two-stream one under the name compress_tiled), but
 * its Triton files still hold the consumers:
 *   ci_decode_tiled_one            rans_decomp_triton_tiled2 / rans_decomp_triton_tiled_splitk
 *                                  (comp_inference/rans_triton.py:355-516)
 *   ci_fused_linear_one            fused_rans_linear_triton_splitk / fused_rans_matmul_kernel_splitk
 *                                  (comp_inference/linear_triton.py:806-1035); workspace:
 *                                  ci_fused_linear_workspace_bytes(M, K, N, th, tw, dense = 1)
 *   ci_fused_embedding_one         fused_rans_embedding_triton_2 / fused_rans_embedding_kernel
 *                                  (comp_inference/embedding_triton.py:8-167)
 *   ci_fused_linear_transposed_one what fused_rans_linear_transposed_triton_2
 *                                  (comp_inference/transposed_linear_triton.py:438-500) is written for;
 *                                  the kernel that function launches is defined nowhere in the reference
 * Arguments as the _ilp2 entry points of the same operator (d_states: tile_width entries a tile).
 * Any tile width; one thread per stream, as for the dense format: format coverage, not a fast path.
 * ------------------------------------------------------------------------------------- */
int ci_encode_tiled_one(const uint8_t *d_symbols, const ci_tiling *t, const uint16_t *h_freqs,
                        const uint16_t *h_cdf, uint8_t *d_scratch, size_t scratch_bytes,
                        uint32_t *d_states, uint32_t *d_sizes, uint32_t *d_tile_offsets,
                        uint32_t *d_tile_max_lens, uint64_t *h_stream_len, ci_stream_t stream);

int ci_pack_tiled_one(const uint8_t *d_scratch, const ci_tiling *t, const uint32_t *d_sizes,
                      const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                      uint8_t *d_stream, uint64_t stream_len, ci_stream_t stream);

int ci_decode_tiled_one(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                        const uint32_t *d_tables, const uint8_t *d_slot_map,
                        const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                        uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width,
                        uint8_t *d_out_exp, const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                        ci_stream_t stream);

int ci_fused_linear_one(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                        const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                        const uint32_t *d_tables, const uint8_t *d_slot_map,
                        const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                        const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                        const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                        void *d_workspace, size_t workspace_bytes, ci_stream_t stream);

int ci_fused_embedding_one(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                           uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                           const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                           const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled, uint32_t K,
                           uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                           uint32_t out_stride, ci_stream_t stream);

int ci_fused_linear_transposed_one(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                   uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                   const uint32_t *d_states, const uint32_t *d_tables,
                                   const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                   const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled,
                                   uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                   uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                   size_t workspace_bytes, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Encoder, flat (legacy) format.  Replaces RansManager::compress (src/cuda/rans_ops.cu:16-72)
 * = StreamConfigurator::suggest (src/cuda/rans_host.cuh:161-183) + kernel rans_compress_kernel
 * (src/cuda/rans_kernels.cuh:393-509).  num_streams = ceil(K / min_block_size) * N; stream g
 * covers the 512-row segment g / N of column g % N (the kernel's segment length is fixed at
 * 512 whatever min_block_size says, src/cuda/rans_kernels.cuh:421).  d_checkpoints receives
 * num_streams * 128 u64 entries: {state, bytes written} before symbols 0, 128, 256, 384 of each
 * segment at [(i / 128) * num_streams + g], zero elsewhere.  ci_pack_flat writes byte j of
 * stream g at [j * num_streams + g], max_len rows (src/cuda/rans_ops.cu:51-65).
 * ------------------------------------------------------------------------------------- */
int ci_flat_geometry(uint32_t K, uint32_t N, uint32_t min_block_size, uint32_t *num_streams,
                     uint32_t *capacity);

int ci_encode_flat(const uint8_t *d_symbols, uint32_t K, uint32_t N, uint32_t num_streams,
                   uint32_t capacity, const uint16_t *h_freqs, const uint16_t *h_cdf,
                   uint8_t *d_scratch, size_t scratch_bytes, uint32_t *d_states, uint32_t *d_sizes,
                   uint64_t *d_checkpoints, uint32_t *h_max_len, ci_stream_t stream);

int ci_pack_flat(const uint8_t *d_scratch, uint32_t num_streams, uint32_t capacity,
                 const uint32_t *d_sizes, uint32_t max_len, uint8_t *d_stream, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Flat decoders.
 * ci_decode_flat_strided replaces the free function decompress() behind ccore.decompress
 * (src/python_bindings.cpp:61-78, src/cuda/rans_ops.cu:619-629, kernel
 * src/cuda/rans_kernels.cuh:626-708): every stream decodes ceil(out_len / num_streams) symbols,
 * symbol i of stream g goes to d_out[g + i * num_streams] (writes past out_len are dropped).
 * ci_decode_flat_segmented replaces rans_decomp_triton (comp_inference/rans_triton.py:172-271):
 * stream g decodes the 512-row segment g / N of column g % N into u8 [K,N].
 * ------------------------------------------------------------------------------------- */
int ci_decode_flat_strided(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                           const uint32_t *d_sizes, uint32_t num_streams, const uint32_t *d_tables,
                           const uint8_t *d_slot_map, uint64_t out_len, uint8_t *d_out,
                           ci_stream_t stream);

int ci_decode_flat_segmented(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                             const uint32_t *d_sizes, uint32_t num_streams, const uint32_t *d_tables,
                             const uint8_t *d_slot_map, uint32_t K, uint32_t N, uint8_t *d_out,
                             ci_stream_t stream);

/* Stand-alone decoder of the dense tiled format (byte order as the reference's fused kernels
 * read it, comp_inference/linear_triton.py:1103-1108, :1147-1170).  Outputs as
 * ci_decode_tiled_ilp2. */
int ci_decode_tiled_dense(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                          const uint32_t *d_tables, const uint8_t *d_slot_map,
                          const uint32_t *d_stream_offsets, const uint32_t *d_stream_sizes,
                          uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width,
                          uint8_t *d_out_exp, const uint8_t *d_man_tiled, uint16_t *d_out_bf16,
                          ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Fused decompress + linear:  out[M,N] (bf16) = x[M,K] (bf16) * W[K,N] (+ bias), W given as
 * coded exponent plane + tile-interleaved raw sign|mantissa plane, never written to memory.
 * ci_fused_linear_ilp2 replaces fused_rans_linear_triton / fused_rans_matmul_kernel_ilp2_splitk
 * (comp_inference/linear_triton.py:229-552); ci_fused_linear_dense replaces
 * fused_rans_linear_triton_uncoalesced (comp_inference/linear_triton.py:1045-1265).
 * x_stride / out_stride are row strides in elements.  d_bias may be NULL.  Products are
 * accumulated in fp32; partial sums over K are combined in a fixed order, so results are
 * reproducible run to run.  d_workspace must hold ci_fused_linear_workspace_bytes(...) bytes
 * (0 for few rows when one workgroup spans all of K); it carries the fp32 split-K partials that
 * the reduction kernel sums (the reference keeps bf16 partials and sums them with torch.sum,
 * comp_inference/linear_triton.py:257-264, :303-314) and, for more than 16 rows of x, a copy of
 * x in the order the matrix cores read it.  A workspace with room for the partials only is
 * accepted: x is then read in place.
 * ------------------------------------------------------------------------------------- */
size_t ci_fused_linear_workspace_bytes(uint32_t M, uint32_t K, uint32_t N, uint32_t tile_height,
                                       uint32_t tile_width, int dense);

int ci_fused_linear_ilp2(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                         const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                         const uint32_t *d_tables, const uint8_t *d_slot_map,
                         const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                         const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                         const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                         void *d_workspace, size_t workspace_bytes, ci_stream_t stream);

int ci_fused_linear_dense(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                          const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                          const uint32_t *d_tables, const uint8_t *d_slot_map,
                          const uint32_t *d_stream_offsets, const uint32_t *d_stream_sizes,
                          const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                          const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                          void *d_workspace, size_t workspace_bytes, ci_stream_t stream);

/* Split-K reduction on its own: d_out[m][n] = bf16(sum_p partial[p][m][n]) (+ bias, added in
 * fp32 and rounded once more, as torch's in-place bf16 add does).  Replaces
 * torch.sum(workspace, dim=0) (+= bias) of comp_inference/linear_triton.py:303-314;
 * partial_is_bf16 != 0 reads the reference's bf16 [P,M,N] workspace layout, 0 reads fp32. */
int ci_splitk_reduce(const void *d_partial, int partial_is_bf16, uint32_t P, uint32_t M, uint32_t N,
                     const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Fused decompress + gather:  out[t, 0..N) (bf16) = table[ids[t], 0..N) for a table [K,N] stored
 * like a weight (K = vocabulary rows, not transposed); ids outside [0,K) give zero rows.
 * ci_fused_embedding_ilp2 replaces fused_rans_embedding_triton / fused_rans_embedding_kernel_ilp2
 * (comp_inference/embedding_triton.py:170-330); ci_fused_embedding_dense replaces
 * fused_rans_embedding_triton_uncoalesced (comp_inference/embedding_triton.py:333-483).
 * d_ids: int64.  out_stride: row stride of d_out in elements.  The default-format entry point
 * sorts the ids on the device and needs ci_fused_embedding_workspace_bytes(...) bytes of
 * scratch (sorted ids, their output rows, one start index per half tile of rows).
 * ------------------------------------------------------------------------------------- */
size_t ci_fused_embedding_workspace_bytes(uint32_t n_ids, uint32_t K, uint32_t tile_height);

int ci_fused_embedding_ilp2(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                            uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                            const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                            const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled, uint32_t K,
                            uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                            uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                            ci_stream_t stream);

int ci_fused_embedding_dense(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                             uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                             const uint8_t *d_slot_map, const uint32_t *d_stream_offsets,
                             const uint32_t *d_stream_sizes, const uint8_t *d_man_tiled, uint32_t K,
                             uint32_t N, uint32_t tile_height, uint32_t tile_width, uint16_t *d_out,
                             uint32_t out_stride, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Fused decompress + linear against a row-per-output weight:  out[M,V] (bf16) = x[M,H] * W^T
 * (+ bias) with W [V,H] stored like an embedding table (tiles of tile_height rows of V by
 * tile_width columns of H).  ci_fused_linear_transposed_ilp2 replaces
 * fused_rans_linear_transposed_triton (comp_inference/transposed_linear_triton.py:187-435);
 * ci_fused_linear_transposed_dense replaces its _uncoalesced variant (:660-883).
 * d_workspace: ci_fused_linear_transposed_workspace_bytes(...) bytes of fp32 partials, one slice
 * per column tile, summed in tile order (the reference zeroes a bf16 workspace and sums it with
 * torch.sum, comp_inference/transposed_linear_triton.py:384, :424-435).
 * ------------------------------------------------------------------------------------- */
size_t ci_fused_linear_transposed_workspace_bytes(uint32_t M, uint32_t H, uint32_t V, uint32_t tile_width);

int ci_fused_linear_transposed_ilp2(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                    uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                    const uint32_t *d_states, const uint32_t *d_tables,
                                    const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                    const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled,
                                    uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                    uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                    size_t workspace_bytes, ci_stream_t stream);

int ci_fused_linear_transposed_dense(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                     uint32_t x_stride, const uint8_t *d_stream, uint64_t stream_len,
                                     const uint32_t *d_states, const uint32_t *d_tables,
                                     const uint8_t *d_slot_map, const uint32_t *d_stream_offsets,
                                     const uint32_t *d_stream_sizes, const uint8_t *d_man_tiled,
                                     uint32_t tile_height, uint32_t tile_width, const uint16_t *d_bias,
                                     uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                     size_t workspace_bytes, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Stand-alone decode of several tensors in one launch (exponent planes only).  No counterpart
 * in the reference, which decodes tensor by tensor (comp_inference/comp_inference.py:633-647):
 * one decode is a chain of tile_height / 2 dependent steps per wavefront however small the
 * tensor, so a model's tensors are best decoded together.  Items are plain host structs.
 * ------------------------------------------------------------------------------------- */
typedef struct ci_decode_item {
    const uint8_t *d_stream;
    uint64_t stream_len;
    const uint32_t *d_states;
    const uint32_t *d_tables;
    const uint8_t *d_slot_map;
    const uint32_t *d_tile_offsets;
    const uint32_t *d_tile_max_lens;
    uint32_t K, N, tile_height, tile_width;
    uint8_t *d_out_exp;
    const void *d_checkpoints; /* NULL, or the index made by ci_build_checkpoints_ilp2 for `segments` */
    uint32_t segments;         /* 0 or 1: whole streams */
} ci_decode_item;

int ci_decode_tiled_ilp2_batch(const ci_decode_item *h_items, uint32_t n_items, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Decoder checkpoints and the fused linear that uses them.  No counterpart in the reference for the
 * tiled format (its flat format records a checkpoint every 128 symbols, src/cuda/rans_kernels.cuh:454-465).
 * A stream of the tiled format is a chain of tile_height / 2 dependent decode steps, and a weight
 * with few tiles (a 4096 x 4096 projection has two per CU) is bound by the length of that chain, not
 * by the chip.  ci_build_checkpoints_ilp2 walks every stream once and records, at `segments` evenly
 * spaced rows, the decoder's state and byte position: an index kept beside the compressed weight
 * (ci_checkpoint_bytes bytes, 8 per stream and checkpoint; the stream is untouched, so the weight stays
 * readable by the reference).  ci_fused_linear_ilp2_segmented then gives every segment of every
 * tile its own wavefront.  tile_width must be 32 and tile_height / 2 a multiple of 16 * segments
 * (for ci_build_checkpoints_ilp2 itself any segment count that divides tile_height / 2 will do);
 * ci_suggest_segments returns 1, 2, 4 or 8 for a weight's shape (1: enough tiles of its own).
 * M above 64, or segments == 1, behaves as ci_fused_linear_ilp2.
 * ------------------------------------------------------------------------------------- */
size_t ci_checkpoint_bytes(uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width, uint32_t segments);

uint32_t ci_suggest_segments(uint32_t K, uint32_t N, uint32_t tile_height, uint32_t tile_width);

int ci_build_checkpoints_ilp2(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                              const uint32_t *d_tables, const uint8_t *d_slot_map,
                              const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens, uint32_t K,
                              uint32_t N, uint32_t tile_height, uint32_t tile_width, uint32_t segments,
                              void *d_checkpoints, size_t checkpoint_bytes, ci_stream_t stream);

size_t ci_fused_linear_workspace_bytes_segmented(uint32_t M, uint32_t K, uint32_t N, uint32_t tile_height,
                                                 uint32_t tile_width, int dense, uint32_t segments);

int ci_fused_linear_ilp2_segmented(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                                   const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                   const uint32_t *d_tables, const uint8_t *d_slot_map,
                                   const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens,
                                   const uint8_t *d_man_tiled, uint32_t tile_height, uint32_t tile_width,
                                   const void *d_checkpoints, uint32_t segments, const uint16_t *d_bias,
                                   uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                                   size_t workspace_bytes, ci_stream_t stream);

/* The gather with decoder checkpoints (any segment count that divides tile_height / 2): a requested row
 * costs at most tile_height / (2 segments) decode steps instead of tile_height / 2. */
size_t ci_fused_embedding_workspace_bytes_segmented(uint32_t n_ids, uint32_t K, uint32_t tile_height,
                                                    uint32_t segments);

int ci_fused_embedding_ilp2_segmented(const int64_t *d_ids, uint32_t n_ids, const uint8_t *d_stream,
                                      uint64_t stream_len, const uint32_t *d_states, const uint32_t *d_tables,
                                      const uint8_t *d_slot_map, const uint32_t *d_tile_offsets,
                                      const uint32_t *d_tile_max_lens, const uint8_t *d_man_tiled, uint32_t K,
                                      uint32_t N, uint32_t tile_height, uint32_t tile_width,
                                      const void *d_checkpoints, uint32_t segments, uint16_t *d_out,
                                      uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                      ci_stream_t stream);

/* The stand-alone decode with decoder checkpoints (tile_width 32, tile_height / 2 a multiple of
 * 16 * segments): every segment of every stream is a work item of its own, so a tensor with few tiles
 * is no longer a chain of tile_height / 2 steps per wavefront, and a batch of tensors ends on short
 * items instead of long ones.  Same output as ci_decode_tiled_ilp2, byte for byte.  Other tile widths
 * ignore the checkpoints.  In a batch, set d_checkpoints / segments per item (ci_decode_item). */
int ci_decode_tiled_ilp2_segmented(const uint8_t *d_stream, uint64_t stream_len, const uint32_t *d_states,
                                   const uint32_t *d_tables, const uint8_t *d_slot_map,
                                   const uint32_t *d_tile_offsets, const uint32_t *d_tile_max_lens, uint32_t K,
                                   uint32_t N, uint32_t tile_height, uint32_t tile_width,
                                   const void *d_checkpoints, uint32_t segments, uint8_t *d_out_exp,
                                   const uint8_t *d_man_tiled, uint16_t *d_out_bf16, ci_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * A compressed weight as one descriptor with the length of every array in it.  The entry points
 * that take it check those lengths against the shape on the host before anything is launched
 * (CI_ERR_ARG), where the bare-pointer entry points above trust the caller: a kernel indexes
 * states by stream, tile metadata by tile, the sign|mantissa plane by tile and row, checkpoints by
 * (tile, segment, stream), and a short array would be read out of bounds on the GPU.  The operands are
 * those of the reference's fused_rans_linear_triton (comp_inference/linear_triton.py:229-246), which
 * passes torch tensors and checks nothing.  Default format only (two streams per column).
 *
 * What the arrays CONTAIN is not checked and need not be trusted for memory safety: with every length in
 * order, no kernel forms a global address from a value it read -- a tile body that would end past
 * stream_len is taken as empty, a checkpoint's position is clamped to its tile body and to the item's
 * window, table lookups are masked to the table -- so a damaged file gives wrong numbers, never an access
 * outside the arrays (d_tile_offsets should be multiples of 16, as an encoder writes them; others cost
 * unaligned loads).
 *
 * d_checkpoints / segments: NULL / 0 or 1, or the index made by ci_build_checkpoints_ilp2.
 * d_slot_table: NULL, or the 32 KB made by ci_build_slot_table; a kernel then copies the table
 * instead of building it from d_tables and d_slot_map in every workgroup.
 * ------------------------------------------------------------------------------------- */
typedef struct ci_tiled_weight {
    uint32_t K, N, tile_height, tile_width;
    const uint8_t *d_stream;
    uint64_t stream_len;              /* bytes */
    const uint32_t *d_states;
    uint64_t n_states;                /* >= tiles * 2 * tile_width */
    const uint32_t *d_tables;         /* 256 entries */
    const uint8_t *d_slot_map;        /* 4096 entries, 4-byte aligned */
    const uint32_t *d_tile_offsets;
    const uint32_t *d_tile_max_lens;
    uint64_t n_tiles;                 /* entries in each of the two, >= tiles */
    const uint8_t *d_man_tiled;       /* NULL (with man_len 0): exponent plane only */
    uint64_t man_len;                 /* bytes, >= tiles * tile_height * tile_width */
    const void *d_checkpoints;
    uint64_t checkpoint_bytes;        /* == ci_checkpoint_bytes(K, N, tile_height, tile_width, segments) */
    uint32_t segments;
    const void *d_slot_table;
    uint64_t slot_table_bytes;        /* == CI_SLOT_TABLE_BYTES when d_slot_table is given */
    uint32_t max_window_rows;         /* 0 (not known), or what ci_max_window_rows wrote for these arrays */
} ci_tiled_weight;

#define CI_SLOT_TABLE_BYTES 32768

/* CI_OK if every array of the descriptor is present, aligned and long enough for its shape.  Runs on
 * the host alone (no device needed). */
int ci_tiled_weight_check(const ci_tiled_weight *w);

/* The decoder's lookup table as the kernels keep it in LDS (one 8-byte entry per 12-bit slot: the
 * reference's slot_map and tables folded into one read, src/cuda/rans_kernels.cuh:677-690), written to
 * d_slot_table (CI_SLOT_TABLE_BYTES, 16-byte aligned).  Derived data kept beside the weight, like the
 * checkpoints. */
int ci_build_slot_table(const uint32_t *d_tables, const uint8_t *d_slot_map, void *d_slot_table,
                        size_t slot_table_bytes, ci_stream_t stream);

/* The largest number of rows of a tile body that one item -- a segment of the 64 streams of a tile, or
 * the whole streams without checkpoints -- reads, written to *d_rows (device memory, 4 bytes) on `stream`;
 * over the items whose 64 streams all have the segment's full length (an item at a ragged edge of the
 * shape is read in place by every kernel, whatever its window), and at least 1.
 * Derived data like the checkpoints: computed once per weight, copied back by the caller and kept in
 * ci_tiled_weight::max_window_rows.  With it the fused linear knows before the launch that every item
 * fits its staging area and runs a kernel without the guarded path; with 0 there it runs the kernel that
 * checks every item.  A value smaller than the true one makes the kernel leave out the items that do not
 * fit (wrong sums, no out-of-bounds access). */
int ci_max_window_rows(const ci_tiled_weight *w, uint32_t *d_rows, ci_stream_t stream);

/* Fused decompress-GEMV/GEMM on a descriptor: what ci_fused_linear_ilp2 / _segmented compute, with the
 * lengths checked.  Workspace: ci_fused_linear_workspace_bytes_segmented(M, K, N, tile_height,
 * tile_width, 0, segments) bytes. */
int ci_fused_linear_tiled(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M, uint32_t x_stride,
                          const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride, void *d_workspace,
                          size_t workspace_bytes, ci_stream_t stream);

/* The other operators on a descriptor, lengths checked before the launch like ci_fused_linear_tiled:
 * ci_decode_tiled = ci_decode_tiled_ilp2[_segmented] (exponent plane to d_out_exp, or, with d_out_bf16
 * given, the bf16 tensor from the weight's own sign|mantissa plane; a descriptor with d_man_tiled NULL and
 * man_len 0 is accepted for the exponent plane alone), ci_fused_embedding_tiled =
 * ci_fused_embedding_ilp2[_segmented] (workspace: ci_fused_embedding_workspace_bytes_segmented),
 * ci_fused_linear_transposed_tiled = ci_fused_linear_transposed_ilp2 with the weight stored [V, H]
 * (K = V rows, N = H columns in the descriptor). */
int ci_decode_tiled(const ci_tiled_weight *w, uint8_t *d_out_exp, uint16_t *d_out_bf16, ci_stream_t stream);

int ci_fused_embedding_tiled(const ci_tiled_weight *w, const int64_t *d_ids, uint32_t n_ids, uint16_t *d_out,
                             uint32_t out_stride, void *d_workspace, size_t workspace_bytes, ci_stream_t stream);

int ci_fused_linear_transposed_tiled(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M, uint32_t x_stride,
                                     const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                     void *d_workspace, size_t workspace_bytes, ci_stream_t stream);

/* The same fused linear for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation.  It has no counterpart in the
 * reference (whose fused_rans_linear_triton allocates its split-K workspace through torch on every
 * call, comp_inference/linear_triton.py:258-263).  It calls no hipMalloc / hipFree or other allocating
 * routine and takes no workspace: partial sums and the fragment copy of x go to a fixed array of
 * CI_NOALLOC_SCRATCH_BYTES of device memory inside the library, one copy per GPU, held until the
 * process ends.  Shapes whose workspace (ci_fused_linear_workspace_bytes_segmented) is larger are
 * refused with CI_ERR_CAPACITY.  All calls on one GPU share that GPU's array: calls that overlap in
 * time on one GPU (two streams, two threads) race; calls queued on one stream do not.  Results are
 * bit-identical to ci_fused_linear_tiled. */
#define CI_NOALLOC_SCRATCH_BYTES (16u << 20)
/* Set-up: the address of the array is asked for once per device (hipGetSymbolAddress), which is not a call to make
 * for the first time while a stream is being captured.  ci_fused_linear_noalloc_init does it for the current device;
 * ci_check_device calls it, so a process that has checked its device is ready, and otherwise the first
 * ci_fused_linear_tiled_noalloc on a device does it -- then that first call must come before any capture.  The
 * current device must be the device of `stream` in every call (the array used is the current device's). */
int ci_fused_linear_noalloc_init(void);
int ci_fused_linear_tiled_noalloc(const ci_tiled_weight *w, const uint16_t *d_x, uint32_t M, uint32_t x_stride,
                                  const uint16_t *d_bias, uint16_t *d_out, uint32_t out_stride,
                                  ci_stream_t stream);

/* More than 64 rows of x: with `enable` non-zero the fused linears of the default format decode a tile once per
 * 128 (65..128 rows) or 256 rows of x and feed every eight-row weight fragment to one matrix instruction per
 * group of 32 rows, instead of decoding the weight again for every 64 rows.  Results are bit-identical either
 * way.  Process-wide, off by default; returns the previous setting.  No counterpart in the reference, which
 * decodes once per 16 rows (comp_inference/linear_triton.py:250-266). */
int ci_fused_linear_wide_rows(int enable);

/* One row of x against a weight with decoder checkpoints (the sixteen-wavefront kernel of
 * ci_fused_linear_transposed_tiled): with `enable` non-zero the sums over the hidden dimension are formed on the
 * matrix pipe -- a block's weights transposed by a matrix instruction against a one-hot operand, then multiply-adds
 * inside a lane -- instead of by lane exchanges.  The sum runs in another order (results within the same
 * tolerance, not bit-identical to the other kernels) and 0 x Inf = NaN: a weight with exponent 255 spoils the
 * other rows of its group of 32, so this is for finite weights.  Process-wide, off by default; returns the
 * previous setting.  No counterpart in the reference. */
int ci_fused_linear_transposed_matrix_sums(int enable);

/* ---------------------------------------------------------------------------------------
 * Bounded waits.  One kernel lets a wavefront wait for another inside a workgroup (the fused linear for up to four
 * rows of x hands its column sums to the last wavefront to arrive through LDS).  Such a wait looks at the flag a
 * bounded number of times; a wavefront that gives up records it in a status word in device memory and goes on, so
 * a defect there ends as wrong sums and an error code, never as a kernel that does not finish.  The reference's
 * Triton kernels have no such wait and nothing to report (their split-K sum is a second launch,
 * comp_inference/linear_triton.py:303-314).
 *   ci_device_status     copies the status word of the current device to *h_status, clears it, waits for `stream`,
 *                        and returns CI_ERR_HIP if a bit was set (CI_STATUS_*).  Synchronises: for health checks
 *                        and tests, not for the token loop.
 *   ci_debug_wait_limit  sets the number of looks (default 2^22, about a fifth of a second); returns the previous
 *                        value.  0 makes every such wait give up at once: the give-up path under test.
 * ------------------------------------------------------------------------------------- */
#define CI_STATUS_WAIT_GAVE_UP 1u
int ci_device_status(uint32_t *h_status, ci_stream_t stream);
uint32_t ci_debug_wait_limit(uint32_t looks);

/* ---------------------------------------------------------------------------------------
 * Verification aids: the contraction of the fused kernels applied to a plain (uncompressed) bf16
 * weight.  No counterpart in the reference, whose tests compare the fused kernels with
 * torch.matmul within allclose(1e-2, 1e-2) (tests/test_mat_mul.py:220, :238) -- a bar that a wrong
 * low mantissa bit passes.  These run the same kernels with the same tiling, the same sequence of
 * matrix instructions, partial sums and reductions as ci_fused_linear_ilp2 /
 * ci_fused_linear_transposed_ilp2 for the same (M, K, N, tile shape), but read the weights from
 * d_w instead of decoding them; their output is therefore bit-identical to the fused kernels' on
 * the compressed form of d_w, and a run of a whole model on decompressed weights can be compared
 * token by token.  Slow (no staging, guarded loads); 32-column tiles only.
 *   ci_plain_linear_same_order:             d_w = bf16 [K, N] row-major; segments as given to
 *                                           ci_fused_linear_ilp2_segmented (1 for ci_fused_linear_ilp2);
 *                                           workspace as ci_fused_linear_workspace_bytes_segmented
 *   ci_plain_linear_transposed_same_order:  d_w = bf16 [V, H] row-major; workspace as
 *                                           ci_fused_linear_transposed_workspace_bytes(M, H, V, tw)
 * ------------------------------------------------------------------------------------- */
int ci_plain_linear_same_order(const uint16_t *d_x, uint32_t M, uint32_t K, uint32_t N, uint32_t x_stride,
                               const uint16_t *d_w, uint32_t tile_height, uint32_t tile_width,
                               uint32_t segments, const uint16_t *d_bias, uint16_t *d_out,
                               uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                               ci_stream_t stream);

int ci_plain_linear_transposed_same_order(const uint16_t *d_x, uint32_t M, uint32_t H, uint32_t V,
                                          uint32_t x_stride, const uint16_t *d_w, uint32_t tile_height,
                                          uint32_t tile_width, const uint16_t *d_bias, uint16_t *d_out,
                                          uint32_t out_stride, void *d_workspace, size_t workspace_bytes,
                                          ci_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* COMP_INFERENCE_HIP_H */
