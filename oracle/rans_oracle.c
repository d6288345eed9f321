/*
 * rans_oracle.c -- CPU restatement of the reference's compressed-weight arithmetic.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the parity checker for the HIP kernels and
 * the timed "CPU baseline" leg of bench.py.  Nothing in the shipped package may import,
 * link or call it; the product path runs on the GPU only.
 *
 * Every function cites the reference lines (paths under the reference checkout) whose
 * arithmetic it restates.  The reference has no CPU coder: its encoder and one decoder
 * are CUDA kernels, the other decoders are Triton kernels.  The bodies below are the
 * per-thread arithmetic of those kernels written as plain loops, plus the host-side
 * re-packing that defines the stored stream format.
 *
 * Pinned by (tests/test_oracle_*.py):
 *   - split/merge: exhaustive over all 65536 bf16 patterns, closed form.
 *   - LUT: exact-integer floor cross-check, sum/positivity/scan invariants, uniform and
 *     single-symbol closed forms, argmax tie order.
 *   - coder: decode(encode(x)) == x for every layout; state interval invariant
 *     [2^16, 2^24); decoder ends on 2^16 with every byte consumed; decode_step(encode_step(x, s))
 *     == (x, s); an independent plain-integer encoder and decoder (tests/pyref.py) byte for byte;
 *     closed forms for power-of-two frequencies and a one-symbol input; layout invariants of
 *     the packed stream (offset scan, zero prefix rows, length).
 *   - mantissa interleave: explicit index formula + inverse.
 *   - fused GEMM numerics restatement: compared with float64 matmul within the
 *     reference's own 1e-2/1e-2 tolerance.
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define RO_PROB_BITS 12u
#define RO_PROB_SCALE 4096u
#define RO_PROB_MASK 4095u
#define RO_RANS_L (1u << 16) /* src/cuda/rans.cuh:42-44: 8-bit io => 2^16 */
#define RO_FLAT_SEG 512u     /* src/cuda/rans_kernels.cuh:421 (hard-coded B) */
#define RO_CKPT_INTERVAL 128u /* src/cuda/rans_kernels.cuh:5 */

enum {
    RO_OK = 0,
    RO_ERR_ARG = 1,
    RO_ERR_CAPACITY = 2, /* a stream outgrew the reference's per-stream capacity */
    RO_ERR_NOMEM = 3,
    RO_ERR_CORRUPT = 4
};

/* ------------------------------------------------------------------------------------
 * bf16 plane split / merge
 * comp_inference/comp_inference.py:10-32 (split), :156-180 (merge),
 * comp_inference/rans_triton.py:12-28 (in-kernel merge).
 * exponent plane = bits 14..7; sign|mantissa plane = bit 15 moved to bit 7, bits 6..0.
 * ---------------------------------------------------------------------------------- */
void ro_split_bf16(const uint16_t *w, uint64_t n, uint8_t *exp_plane, uint8_t *man_plane) {
    for (uint64_t i = 0; i < n; ++i) {
        uint32_t raw = w[i];
        exp_plane[i] = (uint8_t)((raw >> 7) & 0xFFu);
        man_plane[i] = (uint8_t)((((raw >> 15) & 1u) << 7) | (raw & 0x7Fu));
    }
}

void ro_merge_bf16(const uint8_t *exp_plane, const uint8_t *man_plane, uint64_t n, uint16_t *w) {
    for (uint64_t i = 0; i < n; ++i) {
        uint32_t m = man_plane[i], e = exp_plane[i];
        w[i] = (uint16_t)(((m & 0x80u) << 8) | (e << 7) | (m & 0x7Fu));
    }
}

/* ------------------------------------------------------------------------------------
 * 12-bit frequency table.  comp_inference/comp_inference.py:183-239.
 * Same float64 expression as numpy evaluates: floor(count / total * 4096), zero -> 1,
 * surplus added to the first maximum, deficit removed one unit at a time from the
 * current first maximum; cdf = exclusive prefix sum.
 * ---------------------------------------------------------------------------------- */
static int first_argmax(const int32_t *f) {
    int best = 0;
    for (int s = 1; s < 256; ++s)
        if (f[s] > f[best]) best = s;
    return best;
}

int ro_get_lut(const uint8_t *data, uint64_t n, uint16_t *freq_out, uint16_t *cdf_out) {
    if (n == 0) return RO_ERR_ARG;
    uint64_t counts[256];
    memset(counts, 0, sizeof counts);
    for (uint64_t i = 0; i < n; ++i) counts[data[i]]++;
    int32_t f[256];
    int64_t sum = 0;
    for (int s = 0; s < 256; ++s) {
        double q = (double)counts[s] / (double)n * 4096.0;
        f[s] = (int32_t)floor(q);
        if (f[s] == 0) f[s] = 1;
        sum += f[s];
    }
    int64_t diff = 4096 - sum;
    if (diff > 0) {
        f[first_argmax(f)] += (int32_t)diff;
    } else {
        while (diff < 0) {
            int a = first_argmax(f);
            f[a] -= 1;
            if (f[a] < 1) return RO_ERR_CORRUPT;
            diff += 1;
        }
    }
    uint32_t run = 0;
    for (int s = 0; s < 256; ++s) {
        cdf_out[s] = (uint16_t)run;
        freq_out[s] = (uint16_t)f[s];
        run += (uint32_t)f[s];
    }
    return run == 4096 ? RO_OK : RO_ERR_CORRUPT;
}

/* ------------------------------------------------------------------------------------
 * Decoder tables.  src/cuda/rans.cuh:10-13 (packed {u16 freq; u16 cdf}),
 * src/cuda/rans_host.cuh:476-488 (slot map = inverse cdf).
 * ---------------------------------------------------------------------------------- */
void ro_build_tables(const uint16_t *freq, const uint16_t *cdf, uint32_t *tables, uint8_t *slot_map) {
    for (int s = 0; s < 256; ++s) {
        tables[s] = (uint32_t)freq[s] | ((uint32_t)cdf[s] << 16);
        for (uint32_t j = 0; j < freq[s]; ++j) {
            uint32_t slot = (uint32_t)cdf[s] + j;
            if (slot < RO_PROB_SCALE) slot_map[slot] = (uint8_t)s;
        }
    }
}

/* ------------------------------------------------------------------------------------
 * One encoder step and one decoder step, shared by every layout.
 * encode: src/cuda/rans_kernels.cuh:123-151 (x_max = ((L>>12)<<8)*freq, byte-wise emit,
 *         then C(x,s) = ((x/f)<<12) + x%f + cdf).
 * decode: src/cuda/rans_kernels.cuh:676-706, comp_inference/rans_triton.py:93-119
 *         (slot, symbol, D(x) = f*(x>>12) + slot - cdf, at most two byte refills).
 * ---------------------------------------------------------------------------------- */
typedef struct {
    uint8_t *buf;
    uint32_t len;
    uint32_t cap;
} ro_bytes;

static inline int enc_step(uint32_t *state, uint32_t f, uint32_t c, ro_bytes *out) {
    uint32_t x = *state;
    const uint32_t x_max = ((RO_RANS_L >> RO_PROB_BITS) << 8) * f;
    while (x >= x_max) {
        if (out->len >= out->cap) return RO_ERR_CAPACITY;
        out->buf[out->len++] = (uint8_t)(x & 0xFFu);
        x >>= 8;
    }
    *state = ((x / f) << RO_PROB_BITS) + (x % f) + c;
    return RO_OK;
}

/* Capacity the reference gives each stream in its temporary buffer
 * (src/cuda/rans_host.cuh:470-471, :207-208): (uint32)(ceil(n/streams) * 1.25) + 64. */
static uint32_t stream_capacity(uint64_t n_symbols, uint32_t n_streams) {
    uint64_t per = (n_symbols + n_streams - 1) / n_streams;
    return (uint32_t)((double)per * 1.25) + 64u;
}

/* ------------------------------------------------------------------------------------
 * Tiled two-streams-per-column ("ILP2") encoder + packing: the default format.
 * kernel:  src/cuda/rans_kernels.cuh:76-188
 * counts:  src/cuda/rans_host.cuh:447-471
 * packing: src/cuda/rans_ops.cu:328-375 (tile-major, rows of 2*tw bytes, every stream
 *          bottom-aligned under max_len with a zero prefix)
 * Streams of columns >= N keep state 2^16 / size 0 here (the reference leaves them
 * uninitialised, src/cuda/rans_kernels.cuh:99-100).
 *
 * Caller provides: states[S], sizes[S], tile_offsets[T], tile_max_lens[T] and receives a
 * malloc'ed stream through *stream_out (free with ro_free).
 * ---------------------------------------------------------------------------------- */
void ro_free(void *p) { free(p); }

/* `halves` streams per column and tile: 2 = the default format above, 1 = one stream over the whole tile
 * height (the reference's first tiled format: kernel src/cuda/rans_kernels.cuh:316-391, packing
 * src/cuda/rans_ops.cu:522-566, the same interleave with rows of tw bytes). */
static int encode_tiled(const uint8_t *sym, uint32_t K, uint32_t N, const uint16_t *freq,
                        const uint16_t *cdf, uint32_t th, uint32_t tw, uint32_t halves, uint32_t *states,
                        uint32_t *sizes, uint32_t *tile_offsets, uint32_t *tile_max_lens,
                        uint8_t **stream_out, uint64_t *stream_len_out) {
    if (th == 0 || tw == 0 || (halves == 2 && th % 16 != 0) || K == 0 || N == 0) return RO_ERR_ARG;
    const uint32_t tiles_k = (K + th - 1) / th, tiles_n = (N + tw - 1) / tw;
    const uint32_t T = tiles_k * tiles_n, spt = halves * tw, S = T * spt;
    const uint32_t cap = stream_capacity((uint64_t)K * N, S);
    const uint32_t half = th / halves;
    uint8_t **bodies = (uint8_t **)calloc(T, sizeof(uint8_t *));
    if (!bodies) return RO_ERR_NOMEM;
    int status = RO_OK;

#pragma omp parallel
    {
        uint8_t *tmp = (uint8_t *)malloc((size_t)spt * cap);
#pragma omp for schedule(dynamic, 4)
        for (uint32_t t = 0; t < T; ++t) {
            if (!tmp) {
#pragma omp atomic write
                status = RO_ERR_NOMEM;
                continue;
            }
            const uint32_t tk = t / tiles_n, tn = t % tiles_n, row0 = tk * th;
            uint32_t max_len = 0;
            for (uint32_t q = 0; q < spt; ++q) {
                const uint32_t lane = q % tw, is_b = q / tw;
                const uint32_t col = tn * tw + lane;
                ro_bytes out = {tmp + (size_t)q * cap, 0, cap};
                uint32_t x = RO_RANS_L;
                if (col < N) {
                    const int lo = (int)(is_b * half), hi = lo + (int)half;
                    for (int i = hi - 1; i >= lo; --i) { /* bottom-up */
                        uint32_t row = row0 + (uint32_t)i;
                        if (row >= K) continue;
                        uint32_t s = sym[(size_t)row * N + col];
                        if (enc_step(&x, freq[s], cdf[s], &out) != RO_OK) {
#pragma omp atomic write
                            status = RO_ERR_CAPACITY;
                            break;
                        }
                    }
                }
                states[(size_t)t * spt + q] = x;
                sizes[(size_t)t * spt + q] = out.len;
                if (out.len > max_len) max_len = out.len;
            }
            tile_max_lens[t] = max_len;
            uint8_t *body = (uint8_t *)calloc((size_t)max_len * spt + 1, 1);
            if (!body) {
#pragma omp atomic write
                status = RO_ERR_NOMEM;
                continue;
            }
            for (uint32_t q = 0; q < spt; ++q) {
                const uint32_t len = sizes[(size_t)t * spt + q], pad = max_len - len;
                const uint8_t *src = tmp + (size_t)q * cap;
                for (uint32_t j = 0; j < len; ++j) body[(size_t)(pad + j) * spt + q] = src[j];
            }
            bodies[t] = body;
        }
        free(tmp);
    }

    uint64_t total = 0;
    if (status == RO_OK) {
        for (uint32_t t = 0; t < T; ++t) {
            tile_offsets[t] = (uint32_t)total; /* u32 in the reference too */
            total += (uint64_t)tile_max_lens[t] * spt;
        }
        uint8_t *stream = (uint8_t *)malloc(total ? total : 1);
        if (!stream) status = RO_ERR_NOMEM;
        else {
            uint64_t off = 0;
            for (uint32_t t = 0; t < T; ++t) {
                uint64_t nb = (uint64_t)tile_max_lens[t] * spt;
                memcpy(stream + off, bodies[t], nb);
                off += nb;
            }
            *stream_out = stream;
            *stream_len_out = total;
        }
    }
    for (uint32_t t = 0; t < T; ++t) free(bodies[t]);
    free(bodies);
    return status;
}

int ro_encode_tiled_ilp2(const uint8_t *sym, uint32_t K, uint32_t N, const uint16_t *freq,
                         const uint16_t *cdf, uint32_t th, uint32_t tw, uint32_t *states,
                         uint32_t *sizes, uint32_t *tile_offsets, uint32_t *tile_max_lens,
                         uint8_t **stream_out, uint64_t *stream_len_out) {
    return encode_tiled(sym, K, N, freq, cdf, th, tw, 2, states, sizes, tile_offsets, tile_max_lens, stream_out,
                        stream_len_out);
}

/* One stream per column and tile, packed into tile bodies (src/cuda/rans_kernels.cuh:316-391,
 * src/cuda/rans_ops.cu:412-600): T * tw streams. */
int ro_encode_tiled_one(const uint8_t *sym, uint32_t K, uint32_t N, const uint16_t *freq,
                        const uint16_t *cdf, uint32_t th, uint32_t tw, uint32_t *states,
                        uint32_t *sizes, uint32_t *tile_offsets, uint32_t *tile_max_lens,
                        uint8_t **stream_out, uint64_t *stream_len_out) {
    return encode_tiled(sym, K, N, freq, cdf, th, tw, 1, states, sizes, tile_offsets, tile_max_lens, stream_out,
                        stream_len_out);
}

/* ------------------------------------------------------------------------------------
 * Decoder for the ILP2 format.  comp_inference/rans_triton.py:34-119.
 * Lanes of columns >= N and rows >= K take no step.  end_states (optional, S entries)
 * and bytes_left (optional) expose the final coder state for the invariant tests.
 * ---------------------------------------------------------------------------------- */
static int decode_tiled(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                        const uint32_t *tables, const uint8_t *slot_map,
                        const uint32_t *tile_offsets, const uint32_t *tile_max_lens, uint32_t K,
                        uint32_t N, uint32_t th, uint32_t tw, uint32_t halves, uint8_t *out, uint32_t *end_states,
                        int32_t *rows_left) {
    if (th == 0 || tw == 0 || (halves == 2 && (th & 1u))) return RO_ERR_ARG;
    const uint32_t tiles_k = (K + th - 1) / th, tiles_n = (N + tw - 1) / tw;
    const uint32_t T = tiles_k * tiles_n, spt = halves * tw, half = th / halves;
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 4)
    for (uint32_t t = 0; t < T; ++t) {
        const uint32_t tk = t / tiles_n, tn = t % tiles_n, row0 = tk * th;
        const uint64_t base = tile_offsets[t];
        const uint32_t depth = tile_max_lens[t];
        if (base + (uint64_t)depth * spt > stream_len) {
#pragma omp atomic write
            status = RO_ERR_CORRUPT;
            continue;
        }
        uint32_t x[256];
        int32_t r[256];
        if (spt > 256) {
#pragma omp atomic write
            status = RO_ERR_ARG;
            continue;
        }
        for (uint32_t q = 0; q < spt; ++q) {
            x[q] = states[(size_t)t * spt + q];
            r[q] = (int32_t)depth - 1;
        }
        for (uint32_t i = 0; i < half; ++i) {
            for (uint32_t q = 0; q < spt; ++q) {
                const uint32_t lane = q % tw, is_b = q / tw;
                const uint32_t col = tn * tw + lane, row = row0 + i + is_b * half;
                if (col >= N || row >= K) continue;
                uint32_t xs = x[q];
                const uint32_t slot = xs & RO_PROB_MASK;
                const uint32_t s = slot_map[slot];
                out[(size_t)row * N + col] = (uint8_t)s;
                const uint32_t pk = tables[s];
                xs = (pk & 0xFFFFu) * (xs >> RO_PROB_BITS) + (slot - (pk >> 16));
                for (int pass = 0; pass < 2; ++pass) {
                    if (xs < RO_RANS_L && r[q] >= 0) {
                        xs = (xs << 8) | stream[base + (uint64_t)r[q] * spt + q];
                        r[q] -= 1;
                    }
                }
                x[q] = xs;
            }
        }
        for (uint32_t q = 0; q < spt; ++q) {
            if (end_states) end_states[(size_t)t * spt + q] = x[q];
            if (rows_left) rows_left[(size_t)t * spt + q] = r[q];
        }
    }
    return status;
}

int ro_decode_tiled_ilp2(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                         const uint32_t *tables, const uint8_t *slot_map,
                         const uint32_t *tile_offsets, const uint32_t *tile_max_lens, uint32_t K,
                         uint32_t N, uint32_t th, uint32_t tw, uint8_t *out, uint32_t *end_states,
                         int32_t *rows_left) {
    return decode_tiled(stream, stream_len, states, tables, slot_map, tile_offsets, tile_max_lens, K, N, th, tw, 2, out,
                        end_states, rows_left);
}

/* Decoder for the one-stream-per-column tiled format: comp_inference/rans_triton.py:399-464 (rows of tw bytes,
 * one state per lane, the whole tile height in one chain). */
int ro_decode_tiled_one(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                        const uint32_t *tables, const uint8_t *slot_map,
                        const uint32_t *tile_offsets, const uint32_t *tile_max_lens, uint32_t K,
                        uint32_t N, uint32_t th, uint32_t tw, uint8_t *out, uint32_t *end_states,
                        int32_t *rows_left) {
    return decode_tiled(stream, stream_len, states, tables, slot_map, tile_offsets, tile_max_lens, K, N, th, tw, 1, out,
                        end_states, rows_left);
}

/* ------------------------------------------------------------------------------------
 * Dense ("uncoalesced") tiled format: one stream per (tile, column) over the full tile
 * height, streams concatenated byte-exact.
 * kernel:  src/cuda/rans_kernels.cuh:7-74
 * packing: src/cuda/rans_ops.cu:157-176
 * decode:  comp_inference/linear_triton.py:1103-1108, :1147-1170 (reads offset+idx, idx
 *          from size-1 downwards)
 * ---------------------------------------------------------------------------------- */
int ro_encode_tiled_dense(const uint8_t *sym, uint32_t K, uint32_t N, const uint16_t *freq,
                          const uint16_t *cdf, uint32_t th, uint32_t tw, uint32_t *states,
                          uint32_t *sizes, uint32_t *stream_offsets, uint8_t **stream_out,
                          uint64_t *stream_len_out) {
    if (th == 0 || tw == 0 || K == 0 || N == 0) return RO_ERR_ARG;
    const uint32_t tiles_k = (K + th - 1) / th, tiles_n = (N + tw - 1) / tw;
    const uint32_t T = tiles_k * tiles_n, S = T * tw;
    const uint32_t cap = stream_capacity((uint64_t)K * N, S);
    uint8_t *tmp = (uint8_t *)malloc((size_t)S * cap);
    if (!tmp) return RO_ERR_NOMEM;
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t sid = 0; sid < S; ++sid) {
        const uint32_t t = sid / tw, lane = sid % tw;
        const uint32_t tk = t / tiles_n, tn = t % tiles_n, col = tn * tw + lane;
        ro_bytes out = {tmp + (size_t)sid * cap, 0, cap};
        uint32_t x = RO_RANS_L;
        if (col < N) {
            for (int i = (int)th - 1; i >= 0; --i) {
                uint32_t row = tk * th + (uint32_t)i;
                if (row >= K) continue;
                uint32_t s = sym[(size_t)row * N + col];
                if (enc_step(&x, freq[s], cdf[s], &out) != RO_OK) {
#pragma omp atomic write
                    status = RO_ERR_CAPACITY;
                    break;
                }
            }
        }
        states[sid] = x;
        sizes[sid] = out.len;
    }
    if (status == RO_OK) {
        uint64_t total = 0;
        for (uint32_t sid = 0; sid < S; ++sid) {
            stream_offsets[sid] = (uint32_t)total;
            total += sizes[sid];
        }
        uint8_t *stream = (uint8_t *)malloc(total ? total : 1);
        if (!stream) status = RO_ERR_NOMEM;
        else {
            for (uint32_t sid = 0; sid < S; ++sid)
                memcpy(stream + stream_offsets[sid], tmp + (size_t)sid * cap, sizes[sid]);
            *stream_out = stream;
            *stream_len_out = total;
        }
    }
    free(tmp);
    return status;
}

int ro_decode_tiled_dense(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                          const uint32_t *tables, const uint8_t *slot_map,
                          const uint32_t *stream_offsets, const uint32_t *stream_sizes, uint32_t K,
                          uint32_t N, uint32_t th, uint32_t tw, uint8_t *out, uint32_t *end_states,
                          int32_t *bytes_left) {
    const uint32_t tiles_k = (K + th - 1) / th, tiles_n = (N + tw - 1) / tw;
    const uint32_t S = tiles_k * tiles_n * tw;
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t sid = 0; sid < S; ++sid) {
        const uint32_t t = sid / tw, lane = sid % tw;
        const uint32_t tk = t / tiles_n, tn = t % tiles_n, col = tn * tw + lane;
        uint32_t x = states[sid];
        int32_t idx = (int32_t)stream_sizes[sid] - 1;
        const uint64_t off = stream_offsets[sid];
        if (off + stream_sizes[sid] > stream_len) {
#pragma omp atomic write
            status = RO_ERR_CORRUPT;
            continue;
        }
        if (col < N) {
            for (uint32_t i = 0; i < th; ++i) {
                uint32_t row = tk * th + i;
                if (row >= K) break;
                const uint32_t slot = x & RO_PROB_MASK, s = slot_map[slot], pk = tables[s];
                out[(size_t)row * N + col] = (uint8_t)s;
                x = (pk & 0xFFFFu) * (x >> RO_PROB_BITS) + (slot - (pk >> 16));
                for (int pass = 0; pass < 2; ++pass)
                    if (x < RO_RANS_L && idx >= 0) x = (x << 8) | stream[off + (uint32_t)idx--];
            }
        }
        if (end_states) end_states[sid] = x;
        if (bytes_left) bytes_left[sid] = idx + 1;
    }
    return status;
}

/* ------------------------------------------------------------------------------------
 * Flat (legacy) format.
 * stream count:  src/cuda/rans_host.cuh:161-183 (ceil(K / min_block) * N)
 * kernel:        src/cuda/rans_kernels.cuh:393-509: stream gid = (segment gid/N of 512
 *                rows, column gid%N); checkpoint {state, offset} before symbols
 *                0,128,256,384 of the segment, stored at [(i/128)*streams + gid]
 * packing:       src/cuda/rans_ops.cu:51-65: byte j of stream gid at [j*streams + gid],
 *                trimmed to max_len rows
 * Caller provides states[S], sizes[S], checkpoints[S*128] (u64 = state | offset<<32).
 * ---------------------------------------------------------------------------------- */
uint32_t ro_flat_num_streams(uint32_t K, uint32_t N, uint32_t min_block) {
    if (min_block == 0) return 0;
    return ((K + min_block - 1) / min_block) * N;
}

int ro_encode_flat(const uint8_t *sym, uint32_t K, uint32_t N, const uint16_t *freq,
                   const uint16_t *cdf, uint32_t min_block, uint32_t *states, uint32_t *sizes,
                   uint64_t *checkpoints, uint8_t **stream_out, uint64_t *stream_len_out) {
    const uint32_t S = ro_flat_num_streams(K, N, min_block);
    if (S == 0) return RO_ERR_ARG;
    const uint32_t cap = stream_capacity((uint64_t)K * N, S);
    uint8_t *tmp = (uint8_t *)malloc((size_t)S * cap);
    if (!tmp) return RO_ERR_NOMEM;
    memset(checkpoints, 0, (size_t)S * RO_CKPT_INTERVAL * sizeof(uint64_t));
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t gid = 0; gid < S; ++gid) {
        const uint32_t col = gid % N, seg = gid / N, seg_row0 = seg * RO_FLAT_SEG;
        uint32_t n_here = 0;
        if (seg_row0 < K) n_here = (K - seg_row0 < RO_FLAT_SEG) ? (K - seg_row0) : RO_FLAT_SEG;
        ro_bytes out = {tmp + (size_t)gid * cap, 0, cap};
        uint32_t x = RO_RANS_L;
        for (uint32_t i = 0; i < n_here; ++i) {
            if (i % RO_CKPT_INTERVAL == 0)
                checkpoints[(size_t)(i / RO_CKPT_INTERVAL) * S + gid] =
                    (uint64_t)x | ((uint64_t)out.len << 32);
            uint32_t row = seg_row0 + n_here - 1 - i; /* bottom-up */
            uint32_t s = sym[(size_t)row * N + col];
            if (enc_step(&x, freq[s], cdf[s], &out) != RO_OK) {
#pragma omp atomic write
                status = RO_ERR_CAPACITY;
                break;
            }
        }
        states[gid] = x;
        sizes[gid] = out.len;
    }
    if (status == RO_OK) {
        uint32_t max_len = 0;
        for (uint32_t g = 0; g < S; ++g)
            if (sizes[g] > max_len) max_len = sizes[g];
        uint64_t total = (uint64_t)max_len * S;
        uint8_t *stream = (uint8_t *)calloc(total ? total : 1, 1);
        if (!stream) status = RO_ERR_NOMEM;
        else {
            for (uint32_t g = 0; g < S; ++g)
                for (uint32_t j = 0; j < sizes[g]; ++j)
                    stream[(size_t)j * S + g] = tmp[(size_t)g * cap + j];
            *stream_out = stream;
            *stream_len_out = total;
        }
    }
    free(tmp);
    return status;
}

/* Flat decoder that matches the flat encoder's segment mapping.
 * comp_inference/rans_triton.py:172-240 (row = seg*512 + i, byte j at [j*streams+gid]). */
int ro_decode_flat_segmented(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                             const uint32_t *sizes, uint32_t S, const uint32_t *tables,
                             const uint8_t *slot_map, uint32_t K, uint32_t N, uint8_t *out) {
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t gid = 0; gid < S; ++gid) {
        const uint32_t col = gid % N, seg_row0 = (gid / N) * RO_FLAT_SEG;
        if (seg_row0 >= K) continue;
        const uint32_t n_here = (K - seg_row0 < RO_FLAT_SEG) ? (K - seg_row0) : RO_FLAT_SEG;
        uint32_t x = states[gid];
        int32_t off = (int32_t)sizes[gid] - 1;
        if (sizes[gid] && (uint64_t)(sizes[gid] - 1) * S + gid >= stream_len) {
#pragma omp atomic write
            status = RO_ERR_CORRUPT;
            continue;
        }
        for (uint32_t i = 0; i < n_here; ++i) {
            const uint32_t slot = x & RO_PROB_MASK, s = slot_map[slot], pk = tables[s];
            out[(size_t)(seg_row0 + i) * N + col] = (uint8_t)s;
            x = (pk & 0xFFFFu) * (x >> RO_PROB_BITS) + (slot - (pk >> 16));
            for (int pass = 0; pass < 2; ++pass)
                if (x < RO_RANS_L && off >= 0) {
                    x = (x << 8) | stream[(size_t)off * S + gid];
                    off -= 1;
                }
        }
    }
    return status;
}

/* Flat decoder of the native extension: every stream decodes ceil(out_len/S) symbols and
 * writes symbol i of stream gid at out[gid + i*S].  src/cuda/rans_kernels.cuh:626-708,
 * src/cuda/rans_ops.cu:619-629.  Writes past out_len are dropped here (the reference
 * does not check). */
int ro_decode_flat_strided(const uint8_t *stream, uint64_t stream_len, const uint32_t *states,
                           const uint32_t *sizes, uint32_t S, const uint32_t *tables,
                           const uint8_t *slot_map, uint64_t out_len, uint8_t *out) {
    if (S == 0) return RO_ERR_ARG;
    const uint64_t per = (out_len + S - 1) / S;
    int status = RO_OK;
#pragma omp parallel for schedule(dynamic, 64)
    for (uint32_t gid = 0; gid < S; ++gid) {
        uint32_t x = states[gid];
        int64_t off = (int64_t)sizes[gid] - 1;
        if (sizes[gid] && (uint64_t)(sizes[gid] - 1) * S + gid >= stream_len) {
#pragma omp atomic write
            status = RO_ERR_CORRUPT;
            continue;
        }
        for (uint64_t i = 0; i < per; ++i) {
            const uint32_t slot = x & RO_PROB_MASK, s = slot_map[slot], pk = tables[s];
            uint64_t o = gid + i * S;
            if (o < out_len) out[o] = (uint8_t)s;
            x = (pk & 0xFFFFu) * (x >> RO_PROB_BITS) + (slot - (pk >> 16));
            for (int pass = 0; pass < 2; ++pass)
                if (x < RO_RANS_L && off >= 0) {
                    x = (x << 8) | stream[(size_t)off * S + gid];
                    off -= 1;
                }
        }
    }
    return status;
}

/* ------------------------------------------------------------------------------------
 * Sign|mantissa plane tile interleave.  comp_inference/comp_inference.py:35-93.
 * [K,N] zero-padded to tile multiples, stored at tile_id*th*tw + r*tw + c.
 * ---------------------------------------------------------------------------------- */
uint64_t ro_interleaved_len(uint32_t K, uint32_t N, uint32_t th, uint32_t tw) {
    uint64_t tk = (K + th - 1) / th, tn = (N + tw - 1) / tw;
    return tk * tn * th * tw;
}

void ro_interleave_plane(const uint8_t *plane, uint32_t K, uint32_t N, uint32_t th, uint32_t tw,
                         uint8_t *out) {
    const uint32_t tiles_n = (N + tw - 1) / tw;
    memset(out, 0, ro_interleaved_len(K, N, th, tw));
    for (uint32_t row = 0; row < K; ++row)
        for (uint32_t col = 0; col < N; ++col) {
            uint64_t t = (uint64_t)(row / th) * tiles_n + col / tw;
            out[t * th * tw + (uint64_t)(row % th) * tw + col % tw] = plane[(size_t)row * N + col];
        }
}

void ro_uninterleave_plane(const uint8_t *tiled, uint64_t tiled_len, uint32_t K, uint32_t N,
                           uint32_t th, uint32_t tw, uint8_t *plane) {
    const uint32_t tiles_n = (N + tw - 1) / tw;
    for (uint32_t row = 0; row < K; ++row)
        for (uint32_t col = 0; col < N; ++col) {
            uint64_t t = (uint64_t)(row / th) * tiles_n + col / tw;
            uint64_t idx = t * th * tw + (uint64_t)(row % th) * tw + col % tw;
            /* a truncated tail reads as zero padding (comp_inference.py:76-83) */
            plane[(size_t)row * N + col] = idx < tiled_len ? tiled[idx] : 0;
        }
}

/* ------------------------------------------------------------------------------------
 * bf16 helpers (round-to-nearest-even, as torch / Triton .to(bfloat16))
 * ---------------------------------------------------------------------------------- */
static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u); /* NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

/* ------------------------------------------------------------------------------------
 * Numerics of the reference's fused split-K linear on already-decoded weights.
 * comp_inference/linear_triton.py:364-368 (split ranges of ceil(tiles_k/SPLIT_K) k-tiles),
 * :422-466 (per k: acc += f32(bf16(x*w)), one fp32 accumulator per k-tile added into the
 * split accumulator), :536-552 (split result rounded to bf16), :303-314 (sum over splits
 * accumulated in fp32 and rounded once, then bf16 += bias).
 * x: bf16 [M,K], w: bf16 [K,N] (row-major), out: bf16 [M,N].
 * ---------------------------------------------------------------------------------- */
void ro_linear_reference_numerics(const uint16_t *x, const uint16_t *w, const uint16_t *bias,
                                  uint32_t M, uint32_t K, uint32_t N, uint32_t th,
                                  uint32_t split_k, uint16_t *out) {
    const uint32_t tiles_k = (K + th - 1) / th;
    const uint32_t per_split = (tiles_k + split_k - 1) / split_k;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t m = 0; m < M; ++m)
        for (uint32_t n = 0; n < N; ++n) {
            float total = 0.f;
            for (uint32_t sp = 0; sp < split_k; ++sp) {
                float acc = 0.f;
                uint32_t t0 = sp * per_split, t1 = t0 + per_split;
                if (t1 > tiles_k) t1 = tiles_k;
                for (uint32_t t = t0; t < t1; ++t) {
                    float local = 0.f;
                    /* the kernel walks both half tiles in lock step: step i adds row i of
                     * the top half, then row i of the bottom half */
                    for (uint32_t i = 0; i < th / 2; ++i)
                        for (uint32_t h = 0; h < 2; ++h) {
                            uint32_t k = t * th + h * (th / 2) + i;
                            if (k >= K) continue;
                            float p = bf16_to_f32(x[(size_t)m * K + k]) *
                                      bf16_to_f32(w[(size_t)k * N + n]);
                            local += bf16_to_f32(f32_to_bf16(p));
                        }
                    acc += local;
                }
                total += bf16_to_f32(f32_to_bf16(acc));
            }
            uint16_t r = f32_to_bf16(total);
            if (bias) r = f32_to_bf16(bf16_to_f32(r) + bf16_to_f32(bias[n]));
            out[(size_t)m * N + n] = r;
        }
}

/* Plain fp32-accumulate x[M,K] * w[K,N] on bf16 inputs (what torch.matmul is compared to). */
void ro_linear_f32(const uint16_t *x, const uint16_t *w, uint32_t M, uint32_t K, uint32_t N,
                   float *out) {
#pragma omp parallel for schedule(static)
    for (uint32_t m = 0; m < M; ++m) {
        float *o = out + (size_t)m * N;
        for (uint32_t n = 0; n < N; ++n) o[n] = 0.f;
        for (uint32_t k = 0; k < K; ++k) {
            float xv = bf16_to_f32(x[(size_t)m * K + k]);
            const uint16_t *wr = w + (size_t)k * N;
            for (uint32_t n = 0; n < N; ++n) o[n] += xv * bf16_to_f32(wr[n]);
        }
    }
}

/* ------------------------------------------------------------------------------------
 * Fused gather restated literally: per (token, column tile) pick the half stream, take
 * row % (th/2) discarded decode steps, then emit one row.
 * comp_inference/embedding_triton.py:170-275.  ids outside [0,K) give zeros (:204-210).
 * ---------------------------------------------------------------------------------- */
int ro_embedding_gather(const int64_t *ids, uint32_t n_ids, const uint8_t *stream,
                        const uint32_t *states, const uint32_t *tables, const uint8_t *slot_map,
                        const uint32_t *tile_offsets, const uint32_t *tile_max_lens,
                        const uint8_t *man_tiled, uint32_t K, uint32_t N, uint32_t th, uint32_t tw,
                        uint16_t *out) {
    const uint32_t tiles_n = (N + tw - 1) / tw, half = th / 2, spt = 2 * tw;
#pragma omp parallel for collapse(2) schedule(dynamic, 8)
    for (uint32_t m = 0; m < n_ids; ++m)
        for (uint32_t tn = 0; tn < tiles_n; ++tn) {
            int64_t tok = ids[m];
            for (uint32_t lane = 0; lane < tw; ++lane) {
                uint32_t col = tn * tw + lane;
                if (col >= N) continue;
                if (tok < 0 || tok >= (int64_t)K) {
                    out[(size_t)m * N + col] = 0;
                    continue;
                }
                uint32_t tk = (uint32_t)tok / th, rel = (uint32_t)tok % th;
                uint32_t is_b = rel >= half, target = rel % half;
                uint32_t t = tk * tiles_n + tn, q = (is_b ? tw : 0) + lane;
                uint64_t base = tile_offsets[t];
                int32_t r = (int32_t)tile_max_lens[t] - 1;
                uint32_t x = states[(size_t)t * spt + q];
                for (uint32_t i = 0; i < target; ++i) {
                    uint32_t slot = x & RO_PROB_MASK, pk = tables[slot_map[slot]];
                    x = (pk & 0xFFFFu) * (x >> RO_PROB_BITS) + (slot - (pk >> 16));
                    for (int pass = 0; pass < 2; ++pass)
                        if (x < RO_RANS_L && r >= 0) {
                            x = (x << 8) | stream[base + (uint64_t)r * spt + q];
                            r -= 1;
                        }
                }
                uint32_t e = slot_map[x & RO_PROB_MASK];
                uint32_t mb = man_tiled[(uint64_t)t * th * tw + (uint64_t)rel * tw + lane];
                out[(size_t)m * N + col] = (uint16_t)(((mb & 0x80u) << 8) | (e << 7) | (mb & 0x7Fu));
            }
        }
    return RO_OK;
}
