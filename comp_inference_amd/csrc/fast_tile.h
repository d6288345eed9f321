// Hand-scheduled gfx950 inner loops for the default format (32-column tiles, body staged in LDS).
//
// State representation inside these loops
//   X   = 8 * rANS state.  Bits 3..14 are the slot, bits 15.. the quotient; the low three bits
//         carry nothing (renormalisation may leave byte fragments there, every consumer masks
//         or shifts them away).  With this scaling the LDS address of the 8-byte slot-table
//         entry is X & 0x7ff8: one instruction on the serial chain instead of two.
//   tab = slot table with .x = 8*freq | symbol << 24, .y = 8*(slot - cdf), at LDS address 0.
//   q   = LDS address of the next byte of this lane's stream.  The tile body is staged transposed
//         (each lane's bytes contiguous, ascending with the stored row), so consuming a byte is q -= 1.
//   n1  = that byte, read one step ahead.
//
// t = freq * (X >> 15) + bias needs 0, 1 or 2 more bytes (t >= 2^16, t < 2^16, t < 2^8 in unscaled
// terms).  The lanes that need one take it under an execution mask (X = t << 8 | n1, q -= 1, next
// byte requested); needing two takes a symbol of frequency < 16 and is rare, so that case leaves the
// straight line: one compare says whether any lane is still below 2^16, and only then a branch is
// taken to the code that waits for the byte just requested and repeats the step for those lanes.
// Eight VALU instructions and two LDS reads per symbol; the serial chain is v_and -> ds_read_b64 ->
// v_mad_u32_u24 -> v_cmp -> v_lshl_or; the rest sits in the latency shadow of the table read.
//
// Inline-asm rule kept throughout: no LDS or global load issued inside an asm statement is
// still in flight when the statement ends (the compiler does not know about them and may
// reuse or copy their destination registers).
#pragma once
#include "rans_device.h"

namespace ci {

constexpr uint32_t kFastStride = 228;  // bytes of LDS per lane (57 dwords: odd, so lanes spread over banks)
constexpr uint32_t kFastStageBytes = 64 * kFastStride;

// Slot table for the scaled state (see above).  Frequencies are at most 4096, so 8*freq fits
// the 24-bit multiplier with the symbol parked in the top byte.
__device__ __forceinline__ void build_slot_table_x8(uint2 *tab, const uint32_t *__restrict__ tables,
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
            tab[slot] = make_uint2(((pk & 0xFFFFu) << 3) | (s << 24), (slot - (pk >> 16)) << 3);
        }
    }
}

// Stage a tile body (rows of 64 bytes, row r at src + 64 r) into LDS transposed:
// dst[lane * kStride + r] = src[64 r + lane].  A lane fetches 8 columns of two neighbouring rows per
// pass and writes the 8 row pairs as 16-bit LDS stores (LDS instructions, not VALU work, bound these
// kernels: byte stores would be twice as many), so strides are even.  Split in two so that the
// global loads of a group of eight passes (128 rows) are all issued before the first is needed and
// other work -- the slot-table build -- can run under them: stage_fetch issues the loads,
// stage_commit writes LDS.
constexpr int kStagePasses = 8;                       // 16 rows per pass, 128 rows per group
constexpr int kStageGroups = (kFastStride + 127) / 128;
constexpr int stage_groups(uint32_t stride) { return (int)((stride + 127) / 128); }
struct StageRegs {
    uint2 v[kStagePasses][2];  // [pass][row of the pair]: 8 columns each
};

// `row0` = first row of the group (a multiple of 128).
__device__ __forceinline__ void stage_fetch(StageRegs &regs, const uint8_t *__restrict__ src, uint32_t row0,
                                            uint32_t depth, int lane) {
    const uint32_t g = lane & 7, rp = lane >> 3;
#pragma unroll
    for (int p = 0; p < kStagePasses; ++p) {
        const uint32_t r = row0 + p * 16 + 2 * rp;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            regs.v[p][h] = make_uint2(0u, 0u);
            if (r + h < depth) regs.v[p][h] = *reinterpret_cast<const uint2 *>(src + (size_t)(r + h) * 64 + g * 8);
        }
    }
}

// `depth` may differ between lanes (two bodies side by side): rows at or past it are not written,
// except that the odd row of a pair is written with a zero when the even one is the last.
template <uint32_t kStride = kFastStride>
__device__ __forceinline__ void stage_commit(const StageRegs &regs, uint8_t *dst, uint32_t row0, uint32_t depth,
                                             int lane) {
    static_assert(kStride % 2 == 0, "16-bit LDS stores want even column strides");
    const uint32_t g = lane & 7, rp = lane >> 3;
#pragma unroll
    for (int p = 0; p < kStagePasses; ++p) {
        const uint32_t r = row0 + p * 16 + 2 * rp;
        if (r < depth) {
            uint16_t *d = reinterpret_cast<uint16_t *>(dst + (g * 8) * kStride + r);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t lo = j < 4 ? regs.v[p][0].x : regs.v[p][0].y, hi = j < 4 ? regs.v[p][1].x : regs.v[p][1].y;
                // byte j&3 of the even row below byte j&3 of the odd row
                d[j * (kStride / 2)] = (uint16_t)__builtin_amdgcn_perm(hi, lo, 0x0C0C0400u + (j & 3) * 0x0101u);
            }
        }
    }
}

// Stage the `hsel` halves (32 columns each) of two tile bodies side by side, transposed: LDS column
// side * 32 + c holds column hsel * 32 + c of body `side`, one byte per stored row.  Same lane
// roles as stage_fetch / stage_commit: lane = 8 * (row pair) + (8-column group), groups 0..3 = body
// A, 4..7 = body B.
__device__ __forceinline__ void stage_fetch_pair(StageRegs &regs, const uint8_t *__restrict__ src_a, uint32_t depth_a,
                                                 const uint8_t *__restrict__ src_b, uint32_t depth_b, uint32_t hsel,
                                                 uint32_t row0, int lane) {
    const uint32_t g = lane & 7, rp = lane >> 3;
    const uint8_t *src = (g < 4 ? src_a : src_b) + hsel * 32 + (g & 3) * 8;
    const uint32_t depth = g < 4 ? depth_a : depth_b;
#pragma unroll
    for (int p = 0; p < kStagePasses; ++p) {
        const uint32_t r = row0 + p * 16 + 2 * rp;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            regs.v[p][h] = make_uint2(0u, 0u);
            if (r + h < depth) regs.v[p][h] = *reinterpret_cast<const uint2 *>(src + (size_t)(r + h) * 64);
        }
    }
}

// Maximum of a signed value over the 64 lanes of the wavefront (every lane must be active): four DPP
// steps inside each row of 16 lanes, then the four row results.
__device__ __forceinline__ int32_t wave_max_i32(int32_t v) {
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xF, 0xF, false));  // row_half_mirror
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xF, 0xF, false));  // row_mirror
    return max(max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
               max(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}
__device__ __forceinline__ int32_t wave_min_i32(int32_t v) { return -wave_max_i32(-v); }

// ---- workgroups resident for a whole launch ------------------------------------------------------
// The kernels built on the loops below are bound by wavefronts in flight, not by memory: the whole
// LDS goes to the slot table plus as many transposed tile bodies as fit, one workgroup per CU, and
// every wavefront walks a list of tiles.  How many bodies fit depends on the deepest body among the
// workgroup's tiles: 12 wavefronts x 164 bytes per lane (segments of streams, shallow bodies), 11 x 186,
// 10 x 204 or 8 x 254.  Twelve is also the most the register file allows (three wavefronts per SIMD
// at 168 VGPRs).
constexpr int kPersistWaves = 12;
constexpr uint32_t kDepthTiny = 164, kDepthShallow = 186, kDepthMedium = 204, kDepthDeep = 254;

// Builds the slot table and classifies the workgroup by the deepest tile body it will meet
// (`deepest` = this thread's maximum over its share of the workgroup's tiles): returns 3 (all below
// kDepthTiny), 0 (all below kDepthShallow), 1 (all below kDepthMedium) or 2.  Contains the only workgroup
// barrier of such a kernel; blockDim.x must be kPersistWaves * 64.
__device__ __forceinline__ uint32_t persist_classify(uint8_t *lds, const uint32_t *__restrict__ tables,
                                                     const uint8_t *__restrict__ slot_map, uint32_t deepest) {
    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    uint32_t *flags = reinterpret_cast<uint32_t *>(lds + kLdsLimit - 64);  // beyond every staging area
    build_slot_table_x8(reinterpret_cast<uint2 *>(lds), tables, slot_map, tid, kPersistWaves * 64);
    const uint32_t mine = (__builtin_amdgcn_ballot_w64(deepest >= kDepthShallow) ? 1u : 0u) |
                          (__builtin_amdgcn_ballot_w64(deepest >= kDepthMedium) ? 2u : 0u) |
                          (__builtin_amdgcn_ballot_w64(deepest >= kDepthTiny) ? 4u : 0u);
    if (lane == 0) flags[wave] = mine;
    __syncthreads();
    uint32_t any = 0;
#pragma unroll
    for (int w = 0; w < kPersistWaves; ++w) any |= flags[w];
    any = (uint32_t)__builtin_amdgcn_readfirstlane((int)any);
    return (any & 2u) ? 2u : (any & 1u) ? 1u : (any & 4u) ? 0u : 3u;
}

// The same for a workgroup that takes the tiles j, j + n_wg, ... of one tensor.
__device__ __forceinline__ uint32_t persist_prologue(uint8_t *lds, const uint32_t *__restrict__ tables,
                                                     const uint8_t *__restrict__ slot_map,
                                                     const uint32_t *__restrict__ tile_max_lens, uint32_t num_tiles,
                                                     uint32_t j, uint32_t n_wg) {
    uint32_t deepest = 0;
    for (uint64_t t = (uint64_t)threadIdx.x * n_wg + j; t < num_tiles; t += (uint64_t)kPersistWaves * 64 * n_wg)
        deepest = max(deepest, tile_max_lens[t]);
    return persist_classify(lds, tables, slot_map, deepest);
}

// Staging area of wavefront `wave` when kWaves wavefronts of kStride bytes per lane share the LDS.
template <int kWaves, uint32_t kStride>
__device__ __forceinline__ uint8_t *persist_stage(uint8_t *lds, int wave) {
    static_assert(kSlotTableBytes + (uint32_t)kWaves * 64u * kStride + 64u <= kLdsLimit, "staging areas exceed the LDS");
    return lds + kSlotTableBytes + (size_t)wave * 64 * kStride;
}

// Stage a whole tile body (depth < kStride rows) for the hand-scheduled loops.
template <uint32_t kStride>
__device__ __forceinline__ void stage_body(uint8_t *stage, const uint8_t *__restrict__ src, uint32_t depth, int lane) {
    StageRegs body;
#pragma unroll
    for (int grp = 0; grp < stage_groups(kStride); ++grp)
        if ((uint32_t)grp * 128 < depth) {
            stage_fetch(body, src, grp * 128, depth, lane);
            stage_commit<kStride>(body, stage, grp * 128, depth, lane);
        }
}

// ---- windows of tile pairs for sixteen wavefronts per CU -----------------------------------------
// Sixteen wavefronts leave each, next to the slot table, 7 KB of LDS: the window of a short item on a pair of
// neighbouring column tiles (one half of each: 32 + 32 streams), staged as the rows lie in memory -- LDS row r
// of the window = the item's 32 bytes of row r of body A, then those of body B, so lane l finds its bytes at
// 64 r + l and its pointer moves by 64 per byte (qdec = 64).
constexpr int kPairSegWaves = 16;
constexpr uint32_t kPairWinRows = 112;
constexpr uint32_t kPairWinBytes = kPairWinRows * 64;
constexpr int kPairWinPieces = (int)(kPairWinRows / 16);  // one 16-byte load per lane covers 16 rows
static_assert(kPairWinRows % 16 == 0 && kSlotTableBytes + kPairSegWaves * kPairWinBytes <= kLdsLimit, "windows exceed the LDS");

// Rows [0, rows) of the window: lane l loads 16 bytes of row 16 g + l / 4 -- body A for l % 4 < 2, body B
// otherwise, columns hsel * 32 + 16 * (l % 2) on -- and writes them where they belong.  A body shorter than
// the window (win_x < rows) repeats its last row: those bytes belong to no lane.
__device__ __forceinline__ void stage_window_pair(uint8_t *stage, const uint8_t *__restrict__ src_a, uint32_t win_a,
                                                  const uint8_t *__restrict__ src_b, uint32_t win_b, uint32_t hsel,
                                                  uint32_t rows, int lane) {
    const uint32_t r0 = lane / 4, side = (lane % 4) / 2, part = lane % 2;
    const uint8_t *src = (side ? src_b : src_a) + hsel * 32 + part * 16;
    const uint32_t win = side ? win_b : win_a;  // >= 1
    u32x4 w[kPairWinPieces];
#pragma unroll
    for (int g = 0; g < kPairWinPieces; ++g) {
        const uint32_t r = min((uint32_t)g * 16 + r0, win - 1);
        w[g] = *reinterpret_cast<const u32x4 *>(src + (size_t)r * 64);
    }
#pragma unroll
    for (int g = 0; g < kPairWinPieces; ++g) {
        const uint32_t r = (uint32_t)g * 16 + r0;
        if (r < rows) *reinterpret_cast<u32x4 *>(stage + r * 64 + side * 32 + part * 16) = w[g];
    }
}

// The window of ONE tile body for the sixteen-wavefront kernels that take both halves of a tile (fused linear, LM
// head): rows [0, rows) of `src` (64 bytes a row) -> LDS as they lie, piece g = bytes [1024 g + 16 lane, + 16).  Every
// lane loads every piece, from the window's first bytes where its own lie outside: loads without conditions can all
// be in flight together.  rows <= kPairWinRows; nothing is read when rows == 0 (an empty body may end the stream).
constexpr int kWinPieces = (int)(kPairWinRows * 64 / 1024);  // 16 bytes per lane each
__device__ __forceinline__ void stage_window(uint8_t *stage, const uint8_t *__restrict__ src, uint32_t rows, int lane) {
    const uint32_t bytes = rows * 64;
    if (bytes == 0) return;
    u32x4 w[kWinPieces];
#pragma unroll
    for (int g = 0; g < kWinPieces; ++g) {
        const uint32_t o = (uint32_t)g * 1024 + lane * 16;
        w[g] = *reinterpret_cast<const u32x4 *>(src + (o < bytes ? o : 0u));
    }
#pragma unroll
    for (int g = 0; g < kWinPieces; ++g) {
        const uint32_t o = (uint32_t)g * 1024 + lane * 16;
        if (o < bytes) *reinterpret_cast<u32x4 *>(stage + o) = w[g];
    }
}

// ---- assembly building blocks ----------------------------------------------------------------
// Fixed temporaries (declared as clobbers by every user):
//   v[72:73], v[74:75]  slot-table entries of the even / odd step of a pair
//   v76 address, v77 quotient, v78 n1 << 3
//   s[20:21] execution mask saved around the masked part of a step
// Operands by name: X q n1 (lane state), L8 (scaled 2^16 in an SGPR), qdec (LDS bytes from one byte of a
// lane's stream down to the next: 1 in a transposed staging area, 64 where body rows are staged as they
// lie in memory).

// Issue the table read and prepare everything that does not depend on it.
#define CI_STEP_ISSUE(E)                       \
    "v_and_b32 v76, 0x7ff8, %[X]\n"           \
    "ds_read_b64 " E ", v76\n"                \
    "v_lshrrev_b32 v77, 15, %[X]\n"           \
    "s_waitcnt lgkmcnt(1)\n"                   \
    "v_lshlrev_b32 v78, 3, %[n1]\n"

// Consume the table entry (ELO/EHI = its two dwords): new state, pointer, next byte.  The lanes whose
// state fell below 2^16 take a byte under an execution mask; the few that are still below it afterwards
// (a symbol of frequency < 16 met a small quotient: about one step in a thousand on bf16 weight exponents)
// take their second byte out of line.
#define CI_STEP_FINISH(ELO, EHI)                        \
    "s_waitcnt lgkmcnt(0)\n"                            \
    "v_mad_u32_u24 %[X], " ELO ", v77, " EHI "\n"     \
    "v_cmp_gt_u32 vcc, %[L8], %[X]\n"                  \
    "s_and_saveexec_b64 s[20:21], vcc\n"               \
    "v_lshl_or_b32 %[X], %[X], 8, v78\n"              \
    "v_subrev_u32 %[q], %[qdec], %[q]\n"                \
    "ds_read_u8 %[n1], %[q]\n"                         \
    "v_cmpx_gt_u32 vcc, %[L8], %[X]\n"                 \
    "s_cbranch_execnz 8f\n"                            \
    "9:\n"                                             \
    "s_mov_b64 exec, s[20:21]\n"                       \
    ".subsection 1\n"                                  \
    "8:\n"                                             \
    "s_waitcnt lgkmcnt(0)\n"                           \
    "v_lshlrev_b32 v78, 3, %[n1]\n"                   \
    "v_lshl_or_b32 %[X], %[X], 8, v78\n"              \
    "v_subrev_u32 %[q], %[qdec], %[q]\n"                \
    "ds_read_u8 %[n1], %[q]\n"                         \
    "s_branch 9b\n"                                    \
    ".subsection 0\n"

// (scc: s_and_saveexec_b64 writes it -- a loop compare the compiler placed before a statement must not be
// trusted after it)
#define CI_STEP_CLOBBERS                                                                                  \
    "vcc", "scc", "s20", "s21", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "memory"

// Two decoded symbols (top bytes of ELO0, ELO1) and their sign|mantissa bytes (byte %[msel] of the
// dwords M0, M1) -> one dword holding two bf16 (first row in the low half).  v83/v112 temporaries.
#define CI_PACK(ELO0, ELO1, M0, M1, WV)                       \
    "v_perm_b32 v83, " ELO1 ", " ELO0 ", %[selE]\n"          \
    "v_lshrrev_b32 v83, 1, v83\n"                           \
    "v_perm_b32 v112, " M1 ", " M0 ", %[msel]\n"              \
    "v_and_or_b32 " WV ", v112, %[mask], v83\n"

// Advance the per-lane load offsets to the block after the current one (wrapping to block 0
// after the last, so the loads stay inside the tile) -- s23 counts the blocks requested so far.
#define CI_NEXT_BLOCK_OFFSETS                  \
    "s_add_u32 s23, s23, 1\n"                  \
    "s_cmp_eq_u32 s23, %[nblk]\n"              \
    "s_cselect_b32 s24, %[wrapM], 0x100\n"     \
    "s_cselect_b32 s25, %[wrapX], %[xstep]\n"  \
    "v_add_u32 %[moff], s24, %[moff]\n"        \
    "v_add_u32 %[xoff], s25, %[xoff]\n"
// the same step for the x rows 32..63 of a 64-row pass
#define CI_NEXT_BLOCK_OFFSETS2 "v_add_u32 %[xoff2], s25, %[xoff2]\n"
#define CI_LOAD_X2(XR2) "global_load_dwordx4 " XR2 ", %[xoff2], %[xbase]\n"

// Sign|mantissa dwords of rows 0..4 / rows 5..7 + the x fragment of one block into buffer
// (M0..M7, XR).
#define CI_LOAD_LO(M0, M1, M2, M3, M4)                              \
    "global_load_dword " M0 ", %[moff], %[mbase]\n"                 \
    "global_load_dword " M1 ", %[moff], %[mbase] offset:32\n"       \
    "global_load_dword " M2 ", %[moff], %[mbase] offset:64\n"       \
    "global_load_dword " M3 ", %[moff], %[mbase] offset:96\n"       \
    "global_load_dword " M4 ", %[moff], %[mbase] offset:128\n"
#define CI_LOAD_HI(M5, M6, M7, XR)                                  \
    "global_load_dword " M5 ", %[moff], %[mbase] offset:160\n"      \
    "global_load_dword " M6 ", %[moff], %[mbase] offset:192\n"      \
    "global_load_dword " M7 ", %[moff], %[mbase] offset:224\n"      \
    "global_load_dwordx4 " XR ", %[xoff], %[xbase]\n"

// Eight decode steps of one block.  C* = registers of the block being decoded, N* = buffer
// being filled for the block after it (which is also the buffer the previous block used).
// TAIL = what runs in the shadow of step 0: nothing for the first block, otherwise the last
// pack of the previous block and its MFMA.
// EXTRA_OFFS / EXTRA_LOAD: nothing, or the offset step and load of a second x fragment.
#define CI_BLOCK(TAIL, EXTRA_OFFS, EXTRA_LOAD, C0, C1, C2, C3, C4, C5, C6, C7, N0, N1, N2, N3, N4, N5, N6, N7, NX) \
    CI_STEP_ISSUE("v[72:73]") TAIL CI_STEP_FINISH("v72", "v73")                                  \
    CI_STEP_ISSUE("v[74:75]") CI_NEXT_BLOCK_OFFSETS EXTRA_OFFS CI_LOAD_LO(N0, N1, N2, N3, N4)    \
    CI_STEP_FINISH("v74", "v75")                                                                 \
    CI_STEP_ISSUE("v[116:117]") "s_waitcnt vmcnt(5)\n" CI_PACK("v72", "v74", C0, C1, "v108")     \
    CI_STEP_FINISH("v116", "v117")                                                               \
    CI_STEP_ISSUE("v[118:119]") CI_LOAD_HI(N5, N6, N7, NX) EXTRA_LOAD CI_STEP_FINISH("v118", "v119") \
    CI_STEP_ISSUE("v[72:73]") CI_PACK("v116", "v118", C2, C3, "v109") CI_STEP_FINISH("v72", "v73") \
    CI_STEP_ISSUE("v[74:75]") CI_STEP_FINISH("v74", "v75")                                       \
    CI_STEP_ISSUE("v[116:117]") CI_PACK("v72", "v74", C4, C5, "v110") CI_STEP_FINISH("v116", "v117") \
    CI_STEP_ISSUE("v[118:119]") CI_STEP_FINISH("v118", "v119")

// Last pack of a block whose buffer is (.., M6, M7, XR) and the block's MFMA.
#define CI_TAIL(M6, M7, XR)                                             \
    CI_PACK("v116", "v118", M6, M7, "v111")                             \
    "s_nop 1\n"                                                         \
    "v_mfma_f32_32x32x16_bf16 %[acc], v[108:111], " XR ", %[acc]\n"
// ... and a second MFMA of the same weights with the x fragment of rows 32..63
#define CI_TAIL2(M6, M7, XR, XR2) \
    CI_TAIL(M6, M7, XR) "v_mfma_f32_32x32x16_bf16 %[acc2], v[108:111], " XR2 ", %[acc2]\n"

// (argument lists are expanded before CI_BLOCK counts them)
#define CI_BLOCK_X(...) CI_BLOCK(__VA_ARGS__)
#define CI_BUF_A "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91"
#define CI_BUF_B "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99"

// Eight decode steps whose weights leave the statement: W0..W3 = four dwords of two bf16 each
// (rows 0/1, 2/3, 4/5, 6/7 of the block), from the sign|mantissa dwords M0..M7 of those rows.
#define CI_BLOCK8_OUT                                                                                      \
    CI_STEP_ISSUE("v[72:73]") CI_STEP_FINISH("v72", "v73")                                                 \
    CI_STEP_ISSUE("v[74:75]") CI_STEP_FINISH("v74", "v75")                                                 \
    CI_STEP_ISSUE("v[116:117]") CI_PACK("v72", "v74", "%[m0]", "%[m1]", "%[w0]") CI_STEP_FINISH("v116", "v117") \
    CI_STEP_ISSUE("v[118:119]") CI_STEP_FINISH("v118", "v119")                                             \
    CI_STEP_ISSUE("v[72:73]") CI_PACK("v116", "v118", "%[m2]", "%[m3]", "%[w1]") CI_STEP_FINISH("v72", "v73")  \
    CI_STEP_ISSUE("v[74:75]") CI_STEP_FINISH("v74", "v75")                                                 \
    CI_STEP_ISSUE("v[116:117]") CI_PACK("v72", "v74", "%[m4]", "%[m5]", "%[w2]") CI_STEP_FINISH("v116", "v117") \
    CI_STEP_ISSUE("v[118:119]") CI_STEP_FINISH("v118", "v119")                                             \
    CI_PACK("v116", "v118", "%[m6]", "%[m7]", "%[w3]")                                                     \
    "s_waitcnt lgkmcnt(0)\n"

// Per-lane decoder state of the hand-scheduled loops.
struct FastLane {
    uint32_t X, q, n1;
    // `stage` = this wave's staging area, q_lane = this lane's stream inside the tile.
    // kStride = bytes of LDS per lane in the staging area (must exceed the tile's depth).
    template <uint32_t kStride = kFastStride>
    __device__ __forceinline__ void init(const uint8_t *stage, uint32_t depth, uint32_t q_lane, uint32_t state) {
        init_at<kStride>(stage, (int32_t)depth, q_lane, state);
    }
    // The same for a lane that starts in the middle of its stream: `have` = staged bytes of this lane's
    // column from its first row up to and including the next unread byte (<= 0: none left; the bytes such
    // a lane prefetches are never used).
    template <uint32_t kStride = kFastStride>
    __device__ __forceinline__ void init_at(const uint8_t *stage, int32_t have, uint32_t q_lane, uint32_t state) {
        X = state << 3;
        have = max(have, 0);  // (a checkpoint read from a damaged file may say anything: no address is formed from it unclamped)
        const uint8_t *col = stage + q_lane * kStride;
        q = (uint32_t)(uintptr_t)col + (uint32_t)have - 1;  // low 32 bits of an LDS pointer are its LDS address
        n1 = have >= 1 ? col[have - 1] : 0;
    }
};

typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Whole-tile loop of the fused linear for M <= 32: `nblocks` (even, >= 2) blocks of 8 rows per
// half tile.  mbase/moff: tile's sign|mantissa plane (uniform base, per-lane byte offset of the
// aligned dword holding this lane's byte of the first row).  xbase/xoff: x (uniform base, per-lane
// byte offset of the first of this lane's 8 consecutive k), xstep = bytes from one block's
// fragment to the next (16 in a plain row of x).  acc accumulates W^T-tile x x^T.
__device__ __forceinline__ void linear_tile_asm(FastLane &st, f32x16_t &acc, uint64_t mbase, uint32_t moff,
                                                uint64_t xbase, uint32_t xoff, uint32_t xstep, uint32_t man_sel,
                                                uint32_t nblocks, uint32_t qdec = 1) {
    const uint32_t wrap_m = 0u - (nblocks - 1) * 256u, wrap_x = 0u - (nblocks - 1) * xstep;
    asm volatile(
        "s_mov_b32 s23, 0\n"
        "s_lshr_b32 s22, %[nblk], 1\n"
        "s_sub_u32 s22, s22, 1\n"
        // block 0 into buffer A
        CI_LOAD_LO("v84", "v85", "v86", "v87", "v88")
        CI_LOAD_HI("v89", "v90", "v91", "v[100:103]")
        CI_BLOCK_X("", "", "", CI_BUF_A, CI_BUF_B, "v[104:107]")
        CI_BLOCK_X(CI_TAIL("v90", "v91", "v[100:103]"), "", "", CI_BUF_B, CI_BUF_A, "v[100:103]")
        "ci_lin_loop%=:\n"
        "s_cmp_eq_u32 s22, 0\n"
        "s_cbranch_scc1 ci_lin_done%=\n"
        CI_BLOCK_X(CI_TAIL("v98", "v99", "v[104:107]"), "", "", CI_BUF_A, CI_BUF_B, "v[104:107]")
        CI_BLOCK_X(CI_TAIL("v90", "v91", "v[100:103]"), "", "", CI_BUF_B, CI_BUF_A, "v[100:103]")
        "s_sub_u32 s22, s22, 1\n"
        "s_branch ci_lin_loop%=\n"
        "ci_lin_done%=:\n"
        "s_waitcnt vmcnt(0) lgkmcnt(0)\n"
        CI_TAIL("v98", "v99", "v[104:107]")
        "s_nop 15\n"
        "s_nop 15\n"
        : [X] "+v"(st.X), [q] "+v"(st.q), [n1] "+v"(st.n1), [acc] "+v"(acc), [moff] "+v"(moff),
          [xoff] "+v"(xoff)
        : [L8] "s"(kRansL << 3), [selE] "s"(0x070C030Cu), [mask] "s"(0x807F807Fu),
          [msel] "v"(man_sel), [mbase] "s"(mbase), [xbase] "s"(xbase), [nblk] "s"(nblocks), [wrapM] "s"(wrap_m),
          [wrapX] "s"(wrap_x), [xstep] "s"(xstep), [qdec] "s"(qdec)
        : CI_STEP_CLOBBERS, "s22", "s23", "s24", "s25", "v83", "v84", "v85", "v86", "v87", "v88",
          "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101",
          "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v116", "v117",
          "v118", "v119");
}

// The same loop for up to 64 rows of x: a second x fragment (rows 32..63, per-lane offset xoff2,
// buffers v[120:123] / v[124:127]) and a second accumulator fed with the same decoded weights.
__device__ __forceinline__ void linear_tile_asm2(FastLane &st, f32x16_t &acc, f32x16_t &acc2, uint64_t mbase,
                                                 uint32_t moff, uint64_t xbase, uint32_t xoff, uint32_t xoff2,
                                                 uint32_t xstep, uint32_t man_sel, uint32_t nblocks, uint32_t qdec = 1) {
    const uint32_t wrap_m = 0u - (nblocks - 1) * 256u, wrap_x = 0u - (nblocks - 1) * xstep;
    asm volatile(
        "s_mov_b32 s23, 0\n"
        "s_lshr_b32 s22, %[nblk], 1\n"
        "s_sub_u32 s22, s22, 1\n"
        // block 0 into buffer A
        CI_LOAD_LO("v84", "v85", "v86", "v87", "v88")
        CI_LOAD_HI("v89", "v90", "v91", "v[100:103]") CI_LOAD_X2("v[120:123]")
        CI_BLOCK_X("", CI_NEXT_BLOCK_OFFSETS2, CI_LOAD_X2("v[124:127]"), CI_BUF_A, CI_BUF_B, "v[104:107]")
        CI_BLOCK_X(CI_TAIL2("v90", "v91", "v[100:103]", "v[120:123]"), CI_NEXT_BLOCK_OFFSETS2,
                   CI_LOAD_X2("v[120:123]"), CI_BUF_B, CI_BUF_A, "v[100:103]")
        "ci_lin2_loop%=:\n"
        "s_cmp_eq_u32 s22, 0\n"
        "s_cbranch_scc1 ci_lin2_done%=\n"
        CI_BLOCK_X(CI_TAIL2("v98", "v99", "v[104:107]", "v[124:127]"), CI_NEXT_BLOCK_OFFSETS2,
                   CI_LOAD_X2("v[124:127]"), CI_BUF_A, CI_BUF_B, "v[104:107]")
        CI_BLOCK_X(CI_TAIL2("v90", "v91", "v[100:103]", "v[120:123]"), CI_NEXT_BLOCK_OFFSETS2,
                   CI_LOAD_X2("v[120:123]"), CI_BUF_B, CI_BUF_A, "v[100:103]")
        "s_sub_u32 s22, s22, 1\n"
        "s_branch ci_lin2_loop%=\n"
        "ci_lin2_done%=:\n"
        "s_waitcnt vmcnt(0) lgkmcnt(0)\n"
        CI_TAIL2("v98", "v99", "v[104:107]", "v[124:127]")
        "s_nop 15\n"
        "s_nop 15\n"
        : [X] "+v"(st.X), [q] "+v"(st.q), [n1] "+v"(st.n1), [acc] "+v"(acc), [acc2] "+v"(acc2),
          [moff] "+v"(moff), [xoff] "+v"(xoff), [xoff2] "+v"(xoff2)
        : [L8] "s"(kRansL << 3), [selE] "s"(0x070C030Cu), [mask] "s"(0x807F807Fu),
          [msel] "v"(man_sel), [mbase] "s"(mbase), [xbase] "s"(xbase), [nblk] "s"(nblocks), [wrapM] "s"(wrap_m),
          [wrapX] "s"(wrap_x), [xstep] "s"(xstep), [qdec] "s"(qdec)
        : CI_STEP_CLOBBERS, "s22", "s23", "s24", "s25", "v83", "v84", "v85", "v86", "v87", "v88",
          "v89", "v90", "v91", "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101",
          "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v116", "v117",
          "v118", "v119", "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127");
}

// Symbol of the step that used table entry ELO -> one byte at obase + off; off advances a row.
#define CI_STORE_SYM(ELO)                                  \
    "v_lshrrev_b32 v83, 24, " ELO "\n"                    \
    "global_store_byte %[off], v83, %[obase]\n"           \
    "v_add_u32 %[off], %[stride], %[off]\n"

// Stand-alone decode of one half tile per lane: `npairs` >= 1 pairs of steps, symbol i stored at
// obase + off + i * stride (bytes).  The store of a symbol sits in the shadow of the next step.
__device__ __forceinline__ void decode_tile_asm(FastLane &st, uint64_t obase, uint32_t off, uint32_t stride,
                                                uint32_t npairs, uint32_t qdec = 1) {
    asm volatile(
        "s_sub_u32 s22, %[npairs], 1\n"
        CI_STEP_ISSUE("v[72:73]") CI_STEP_FINISH("v72", "v73")
        "ci_dec_loop%=:\n"
        "s_cmp_eq_u32 s22, 0\n"
        "s_cbranch_scc1 ci_dec_done%=\n"
        CI_STEP_ISSUE("v[74:75]") CI_STORE_SYM("v72") CI_STEP_FINISH("v74", "v75")
        CI_STEP_ISSUE("v[72:73]") CI_STORE_SYM("v74") CI_STEP_FINISH("v72", "v73")
        "s_sub_u32 s22, s22, 1\n"
        "s_branch ci_dec_loop%=\n"
        "ci_dec_done%=:\n"
        CI_STEP_ISSUE("v[74:75]") CI_STORE_SYM("v72") CI_STEP_FINISH("v74", "v75")
        CI_STORE_SYM("v74")
        // (the stores may still be on their way: they hold no register the compiler could reuse too early, and
        // the next reader of these bytes is another kernel)
        "s_waitcnt lgkmcnt(0)\n"
        : [X] "+v"(st.X), [q] "+v"(st.q), [n1] "+v"(st.n1), [off] "+v"(off)
        : [L8] "s"(kRansL << 3), [obase] "s"(obase), [stride] "s"(stride), [npairs] "s"(npairs), [qdec] "s"(qdec)
        : CI_STEP_CLOBBERS, "s22", "v83");
}

// Eight symbols of this lane's stream as bf16 weights: w[d] = rows 2d (low half) and 2d + 1 of the
// block.  m[r] = aligned dword holding this lane's sign|mantissa byte of row r, man_sel = the
// per-lane byte selector 0x04040000 + (column & 3) * 0x01010101.
__device__ __forceinline__ void decode8_weights_asm(FastLane &st, const uint32_t (&m)[8], uint32_t man_sel,
                                                    uint32_t (&w)[4], uint32_t qdec = 1) {
    asm volatile(CI_BLOCK8_OUT
                 : [X] "+v"(st.X), [q] "+v"(st.q), [n1] "+v"(st.n1), [w0] "=&v"(w[0]),
                   [w1] "=&v"(w[1]), [w2] "=&v"(w[2]), [w3] "=&v"(w[3])
                 : [L8] "s"(kRansL << 3), [selE] "s"(0x070C030Cu), [mask] "s"(0x807F807Fu),
                   [msel] "v"(man_sel), [m0] "v"(m[0]), [m1] "v"(m[1]), [m2] "v"(m[2]), [m3] "v"(m[3]), [m4] "v"(m[4]),
                   [m5] "v"(m[5]), [m6] "v"(m[6]), [m7] "v"(m[7]), [qdec] "s"(qdec)
                 : CI_STEP_CLOBBERS, "v83", "v112", "v116", "v117", "v118", "v119");
}

// Advance the lane's stream by n >= 1 symbols; returns the table word (symbol in the top byte) of
// the last one.  n must be the same for every lane of the wave.
__device__ __forceinline__ uint32_t advance_asm(FastLane &st, uint32_t n, uint32_t qdec = 1) {
    uint32_t e;
    n = (uint32_t)__builtin_amdgcn_readfirstlane((int)n);  // the loop counter is scalar
    asm volatile(
        "s_mov_b32 s22, %[n]\n"
        "ci_adv_loop%=:\n"
        CI_STEP_ISSUE("v[72:73]") CI_STEP_FINISH("v72", "v73")
        "s_sub_u32 s22, s22, 1\n"
        "s_cmp_lg_u32 s22, 0\n"
        "s_cbranch_scc1 ci_adv_loop%=\n"
        "s_waitcnt lgkmcnt(0)\n"
        "v_mov_b32 %[e], v72\n"
        : [X] "+v"(st.X), [q] "+v"(st.q), [n1] "+v"(st.n1), [e] "=&v"(e)
        : [L8] "s"(kRansL << 3), [n] "s"(n), [qdec] "s"(qdec)
        : CI_STEP_CLOBBERS, "s22");
    return e;
}

}  // namespace ci
