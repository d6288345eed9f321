// Device-side building blocks of the rANS decoders (gfx950, wave64).
//
// Coder constants follow the reference's RansConfig8 (src/cuda/rans_host.cuh:22-24,
// src/cuda/rans.cuh:23-52): 8-bit symbols, 12-bit probabilities, byte-wise I/O, 32-bit
// state kept in [2^16, 2^24).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ci {

constexpr uint32_t kProbBits = 12;
constexpr uint32_t kProbScale = 1u << kProbBits;
constexpr uint32_t kProbMask = kProbScale - 1;
constexpr uint32_t kRansL = 1u << 16;
constexpr int kWave = 64;

// Bytes of LDS taken by the fused slot table: one 8-byte entry per slot.
constexpr uint32_t kSlotTableBytes = kProbScale * 8;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// The reference decoder does two dependent lookups per symbol: slot_map[slot] -> symbol,
// tables[symbol] -> {freq, cdf} (src/cuda/rans_kernels.cuh:677-690).  Here both are folded
// into one LDS-resident table indexed by slot, so a decode step is one ds_read_b64 and one
// v_mad_u32_u24:
//   .x = freq | symbol << 24   (the 24-bit multiply ignores the top byte)
//   .y = slot - cdf[symbol]
__device__ __forceinline__ void build_slot_table(uint2 *tab, const uint32_t *__restrict__ tables,
                                                 const uint8_t *__restrict__ slot_map, int tid,
                                                 int nthreads) {
    const uint32_t *sm4 = reinterpret_cast<const uint32_t *>(slot_map);
    for (int g = tid; g < (int)kProbScale / 4; g += nthreads) {
        uint32_t four = sm4[g];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t slot = (uint32_t)g * 4 + j;
            uint32_t s = (four >> (8 * j)) & 0xFFu;
            uint32_t pk = tables[s];
            tab[slot] = make_uint2((pk & 0xFFFFu) | (s << 24), slot - (pk >> 16));
        }
    }
}

// One decode step on the fused table.  Returns the table word whose top byte is the symbol.
__device__ __forceinline__ uint32_t decode_symbol(uint32_t &x, const uint2 *tab) {
    uint2 e = tab[x & kProbMask];
    x = __umul24(e.x, x >> kProbBits) + e.y;
    return e.x;
}

// The same step on the table built for the scaled state X = 8 * state (fast_tile.h); X stays
// scaled.  Renormalisation on a scaled state: see renorm_scaled of the byte sources.
__device__ __forceinline__ uint32_t decode_symbol_scaled(uint32_t &X, const uint2 *tab) {
    uint2 e = tab[(X >> 3) & kProbMask];
    X = __umul24(e.x, X >> (kProbBits + 3)) + e.y;
    return e.x;
}

// Byte source reading the stream where it lies in global memory, with the reference's
// "row >= 0" guard (comp_inference/rans_triton.py:108).  Used when a tile body does not fit
// the LDS staging area.
struct GlobalBytes {
    const uint8_t *base;  // first byte of this lane's column in the tile body
    int32_t row;
    uint32_t row_bytes;
    __device__ __forceinline__ void init(const uint8_t *tile, uint32_t depth, uint32_t rb, uint32_t q) {
        base = tile + q;
        row = (int32_t)depth - 1;
        row_bytes = rb;
    }
    __device__ __forceinline__ void renorm(uint32_t &x) {
        if (x < kRansL && row >= 0) {
            x = (x << 8) | base[(uint32_t)row * row_bytes];
            row -= 1;
        }
    }
    __device__ __forceinline__ void renorm_scaled(uint32_t &X) {
        if (X < (kRansL << 3) && row >= 0) {
            X = (X << 8) | ((uint32_t)base[(uint32_t)row * row_bytes] << 3);
            row -= 1;
        }
    }
};

// Byte source for the dense ("uncoalesced") format: this lane's bytes are contiguous and
// read from the last one downwards (comp_inference/linear_triton.py:1147-1170).
struct DenseBytes {
    const uint8_t *base;
    int32_t idx;
    __device__ __forceinline__ void init(const uint8_t *b, uint32_t size) {
        base = b;
        idx = (int32_t)size - 1;
    }
    __device__ __forceinline__ void renorm(uint32_t &x) {
        if (x < kRansL && idx >= 0) {
            x = (x << 8) | base[idx];
            idx -= 1;
        }
    }
};

// bf16 bit pattern from exponent symbol and sign|mantissa byte
// (comp_inference/rans_triton.py:12-28).
__device__ __forceinline__ uint32_t assemble_bf16(uint32_t sym, uint32_t man) {
    return ((man & 0x80u) << 8) | (sym << 7) | (man & 0x7Fu);
}

}  // namespace ci
