// Prefill W4A16 GEMM on stream-order weights (wstream.h): y[M, N] = bf16(x[M, K] . W), W = bf16_rne((q - z) * s).
//
// Compute-bound.  The weights never pass through LDS: a stream-order cell is the B operand of
// v_mfma_f32_16x16x32_bf16 for four K-steps of 16 columns, so a wave loads the cells of its own columns straight
// into registers (one 128-bit load per cell and lane), dequantises them there to the bf16 values of the dense
// dequant, and multiplies.  Only x goes through LDS.
//
//   workgroup = 4 waves side by side: 256 rows x 4 * 16 NCB columns; every wave owns all 256 rows (16 row tiles)
//               and its own 16 NCB columns, so each weight is dequantised exactly once per workgroup and the x
//               tile is shared.  16 NCB * 4 fp32 accumulators per lane live in AGPRs (NCB = 4: all 256).
//   K loop    = one quantisation group (128 rows of W) per step: the x tile [256][128] is copied global -> LDS
//               (global_load_lds_dwordx4, double buffered) while the previous group multiplies; the cells and
//               scale words of the next group are requested a step ahead; one barrier per group; the A operands
//               are double buffered in registers, one K-step ahead
//   tiles     = column tiles of two widths in one launch, 256-wide ones first, then 192-wide ones
//               (pick_widths()): M = 2048, N = 14336 becomes 8 x (32 tiles of 256 + 32 tiles of 192), and each of
//               the 256 CUs gets one wide and one narrow tile, 1.75 tile times instead of the two full rounds
//               that 448 tiles of 256 x 256 take.
//
// Issue budget (measured with a loop of this kernel's instruction pattern): the MFMA occupies the matrix pipe for
// 16 cycles and the issue port for 8; a wave issues in order, so exactly two VALU instructions fit behind an
// MFMA for free, a third costs 4 cycles, and two dependent VALU instructions back to back stall on top of that.
// Dequantising 8 weights takes 23 instructions, and with 16 row tiles one B operand feeds 16 MFMAs: the 23
// instructions are cut into 12 slots of two independent instructions (DequantSlots), one slot behind each of the
// first 12 MFMAs of the previous operand.  With 8 row tiles (2.9 instructions per MFMA) the same loop is bound by
// the VALU: 128 x 448 tiles measured 288 us against 257 us for 256 x 256 with the same inner loop.
// Every other instruction (LDS read, memory request, s_add, s_nop, s_waitcnt) takes a slot of its own as well.
//
// Where the time goes at M = 2048, K = 4096, N = 14336 (same box, kernel parts compiled out one at a time): MFMAs alone
// 143 us (the accumulators' pro- and epilogue included), with the dequant 153 us, with LDS reads, x tile copy and
// cell loads 203 - 213 us; without the x tile copy 169 us, without the LDS reads 192 us, without the cell loads 194 us.
// The x tile through registers instead (global_load_dwordx4, then ds_write_b128 a K-step later): 216 against 202 us.
//
// Everything in the inner loop is volatile asm: MFMAs with the accumulator tied to one AGPR quad (through the
// builtin the register allocator gives some MFMAs a destination other than their accumulator input and rotates
// tiles through spare registers, copies via VGPRs behind s_nop stalls), and the dequant slots, because volatile
// asm statements keep their source order, which is the only way to hold an exact MFMA / VALU interleaving
// (scheduling barriers do not stop instruction selection from clustering plain arithmetic).  The compiler does not
// know these are MFMAs, so the wait states it would insert are the kernel's business: a B operand is complete 4
// MFMAs before its first use, an accumulator is revisited 16 NCB MFMAs later, and s_nop covers the read of the
// accumulators after the loop.
//
// LDS layout of the x tile: rows of 128 bf16 (256 B, 16 chunks of 16 bytes), chunk c of row r at slot c ^ r % 16.
// One copy instruction of a wave fills 1 KiB linearly (4 rows); lane l = (row l / 16, slot l % 16) fetches chunk
// slot ^ row % 16.  The A operand read of K-step t (lane (lg, ln): row 16 rt + ln, chunk 4 t + lg) then touches 16
// distinct slots over 16 consecutive rows: conflict-free without padding.
//
// Dequant in registers: e = w & 0x0F0F0F0F and o = (w >> 4) & 0x0F0F0F0F put the eight nibbles of a dword into bytes,
// v_cvt_f32_ubyteN converts each, fma(q, s, -z s) equals (q - z) * s exactly ((q - z) has 5 significant bits, s has 8),
// v_cvt_pk_bf16_f32 rounds once.
#include <algorithm>
#include <functional>
#include <mutex>
#include <type_traits>
#include <vector>

#include "common.h"
#include "kernels.h"
#include "wstream.h"

namespace w4a16 {

namespace {

constexpr int kPfThreads = 256;
constexpr int kPfRowTiles = 16;              // row tiles of 16 per wave
constexpr int kPfRows = 16 * kPfRowTiles;    // rows per workgroup tile
constexpr double kPfSlowdown128 = 1.4, kPfSlowdown64 = 2.0;   // time per column of 128- and 64-column tiles against 256

// eight weights of one dword (rows 8 lg .. 8 lg + 7 of the lane's column) as the four registers of a B operand
__device__ __forceinline__ bf16x8 dequant_operand(uint32_t w, float sf, float c0) {
    uint32_t e = w & 0x0F0F0F0Fu;          // nibbles 0, 2, 4, 6 -> rows 0, 4, 1, 5
    uint32_t o = (w >> 4) & 0x0F0F0F0Fu;   // nibbles 1, 3, 5, 7 -> rows 2, 6, 3, 7
    // kept opaque: the compiler would otherwise fold the masks into one v_bfe_u32 per nibble in front of every
    // convert (two instructions per weight) instead of the byte-select converts v_cvt_f32_ubyte0..3 (one)
    asm volatile("" : "+v"(e), "+v"(o));
    const float k0 = fmaf(static_cast<float>(e & 0xFFu), sf, c0), k4 = fmaf(static_cast<float>((e >> 8) & 0xFFu), sf, c0);
    const float k1 = fmaf(static_cast<float>((e >> 16) & 0xFFu), sf, c0), k5 = fmaf(static_cast<float>(e >> 24), sf, c0);
    const float k2 = fmaf(static_cast<float>(o & 0xFFu), sf, c0), k6 = fmaf(static_cast<float>((o >> 8) & 0xFFu), sf, c0);
    const float k3 = fmaf(static_cast<float>((o >> 16) & 0xFFu), sf, c0), k7 = fmaf(static_cast<float>(o >> 24), sf, c0);
    const u32x4 b = {pack_bf16x2(k0, k1), pack_bf16x2(k2, k3), pack_bf16x2(k4, k5), pack_bf16x2(k6, k7)};
    return __builtin_bit_cast(bf16x8, b);
}

// Four MFMAs of one B operand (row tiles 4 Q .. 4 Q + 3) with, behind each of them, one slot of the NEXT operand's
// dequant: dequant_operand cut into 12 slots of two instructions that do not depend on each other (quarters 0..2;
// quarter 3 is MFMAs only).  Two temporaries per parity (a: registers 0 and 2 of the operand, b: 1 and 3) let the
// converts of one register pair overlap the fmas of the other.  One asm statement per quarter: between separate
// asm statements that pass a register on the compiler inserts an s_nop, and with one wave per SIMD every
// instruction, s_nop included, takes one of the four issue slots of an MFMA.
struct DequantSlots {
    uint32_t w;
    float sf, c0;
    uint32_t e, o;
    float a0, a1, b0, b1;
    uint32_t p0, p1, p2, p3;
    __device__ __forceinline__ bf16x8 operand() const { return __builtin_bit_cast(bf16x8, u32x4{p0, p1, p2, p3}); }
};

#define PF_MFMA(c, a, b) "v_mfma_f32_16x16x32_bf16 %" #c ", %" #a ", %" #b ", %" #c "\n\t"

template <int Q>
__device__ __forceinline__ void mfma_quarter(floatx4 &c0, floatx4 &c1, floatx4 &c2, floatx4 &c3, const bf16x8 &a0, const bf16x8 &a1,
                                             const bf16x8 &a2, const bf16x8 &a3, const bf16x8 &b, DequantSlots &d) {
    if constexpr (Q == 3) {
        asm volatile(PF_MFMA(0, 4, 8) PF_MFMA(1, 5, 8) PF_MFMA(2, 6, 8) "v_mfma_f32_16x16x32_bf16 %3, %7, %8, %3"
                     : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3)
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b));
    } else if constexpr (Q == 0) {
        // %4 e, %5 o, %6 a0, %7 a1, %8 b0 | %9..%12 A, %13 B, %14 w, %15 s, %16 -z s
        asm volatile(PF_MFMA(0, 9, 13) "v_and_b32 %4, 0x0f0f0f0f, %14\n\tv_lshrrev_b32 %5, 4, %14\n\t"
                     PF_MFMA(1, 10, 13) "v_and_b32 %5, 0x0f0f0f0f, %5\n\tv_cvt_f32_ubyte0 %6, %4\n\t"
                     PF_MFMA(2, 11, 13) "v_cvt_f32_ubyte2 %7, %4\n\tv_fma_f32 %6, %6, %15, %16\n\t"
                     PF_MFMA(3, 12, 13) "v_fma_f32 %7, %7, %15, %16\n\tv_cvt_f32_ubyte0 %8, %5"
                     : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3), "=&v"(d.e), "=&v"(d.o), "=&v"(d.a0), "=&v"(d.a1), "=&v"(d.b0)
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b), "v"(d.w), "v"(d.sf), "v"(d.c0));
    } else if constexpr (Q == 1) {
        // %4 a0, %5 a1, %6 b0, %7 b1, %8 p0, %9 p1 | %10..%13 A, %14 B, %15 e, %16 o, %17 s, %18 -z s
        asm volatile(PF_MFMA(0, 10, 14) "v_cvt_pk_bf16_f32 %8, %4, %5\n\tv_cvt_f32_ubyte2 %7, %16\n\t"
                     PF_MFMA(1, 11, 14) "v_fma_f32 %6, %6, %17, %18\n\tv_fma_f32 %7, %7, %17, %18\n\t"
                     PF_MFMA(2, 12, 14) "v_cvt_pk_bf16_f32 %9, %6, %7\n\tv_cvt_f32_ubyte1 %4, %15\n\t"
                     PF_MFMA(3, 13, 14) "v_cvt_f32_ubyte3 %5, %15\n\tv_fma_f32 %4, %4, %17, %18"
                     : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3), "+v"(d.a0), "+v"(d.a1), "+v"(d.b0), "=&v"(d.b1), "=&v"(d.p0), "=&v"(d.p1)
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b), "v"(d.e), "v"(d.o), "v"(d.sf), "v"(d.c0));
    } else {
        // %4 a1, %5 b0, %6 b1, %7 p2, %8 p3 | %9..%12 A, %13 B, %14 a0, %15 o, %16 s, %17 -z s
        asm volatile(PF_MFMA(0, 9, 13) "v_fma_f32 %4, %4, %16, %17\n\tv_cvt_f32_ubyte1 %5, %15\n\t"
                     PF_MFMA(1, 10, 13) "v_cvt_pk_bf16_f32 %7, %14, %4\n\tv_cvt_f32_ubyte3 %6, %15\n\t"
                     PF_MFMA(2, 11, 13) "v_fma_f32 %5, %5, %16, %17\n\tv_fma_f32 %6, %6, %16, %17\n\t"
                     PF_MFMA(3, 12, 13) "v_cvt_pk_bf16_f32 %8, %5, %6"
                     : "+a"(c0), "+a"(c1), "+a"(c2), "+a"(c3), "+v"(d.a1), "=&v"(d.b0), "=&v"(d.b1), "=&v"(d.p2), "=&v"(d.p3)
                     : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b), "v"(d.a0), "v"(d.o), "v"(d.sf), "v"(d.c0));
    }
}

__device__ __forceinline__ void mfma_one(floatx4 &acc, const bf16x8 &a, const bf16x8 &b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// Q4NX order: scale word -> scale s and min' (two bf16 halves)
__device__ __forceinline__ void decode_md_q4(uint32_t md, float &sf, float &c0) {
    sf = __builtin_bit_cast(float, md << 16);
    c0 = __builtin_bit_cast(float, md & 0xFFFF0000u);
}

// A wave-uniform pointer pinned to scalar registers: the loads below then take the form "scalar base + 32-bit lane
// offset" and the per-lane part stays one loop-invariant VGPR (left alone the compiler folds the lane offset into
// a 64-bit VGPR base per stream and spends two VGPRs and a 64-bit add on every request).
using gptr = const __attribute__((address_space(1))) char *;
__device__ __forceinline__ gptr scalar_ptr(const char *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    asm volatile("" : "+s"(lo), "+s"(hi));
    return reinterpret_cast<gptr>(((uint64_t)hi << 32) | lo);
}

// p - bytes, kept in scalar registers (and not re-associated into the lane offsets)
__device__ __forceinline__ gptr scalar_sub(gptr p, uint32_t bytes) {
    const uint64_t v = reinterpret_cast<uint64_t>(p) - bytes;
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    asm volatile("" : "+s"(lo), "+s"(hi));
    return reinterpret_cast<gptr>(((uint64_t)hi << 32) | lo);
}

// scale word -> scale s and -z * s (exact: (128 + z) - 128 and an 8 x 8 bit product)
__device__ __forceinline__ void decode_md(uint32_t md, float &sf, float &c0) {
    sf = __builtin_bit_cast(float, md << 16);
    const float nz = __builtin_bit_cast(float, md & 0xFFFF0000u);   // -(128 + z)
    c0 = (nz + 128.0f) * sf;
}

// Gate and up projection in one tile (launch_gemm_prefill_ws_swiglu): a tile of 64 NCB columns holds 32 NCB columns of
// x . W_gate and the same columns of x . W_up, each wave half and half, and leaves as 32 NCB columns of
// bf16(silu(bf16 gate) * bf16 up).  N is the width of that output; the tile grid runs over 2 N columns.
constexpr int kEpiSwigluPair = 16;

struct PfArgs {
    const uint16_t *x;
    const char *w;
    uint16_t *y;
    int M, K, N, G, NB;
    int tiles_m;
    int n_wide, n_narrow;   // column tiles of each width
    const uint16_t *aux;    // operand of the epilogue: residual / gate [M, N], or the RoPE table [positions, head_dim]
    const char *w_up;       // kEpiSwigluPair: the second matrix (the tile's left half multiplies w, its right half w_up)
    int epi;                // kEpi*, or kEpiSwigluPair
    int rope_cols, rope_hd, rope_pos0;
    int band;               // row panels per band of the tile order (pf_tile_of)
    bool q4;                // the matrices are in Q4NX order
};

// One output tile: rows m0 .., columns col0 .. col0 + 64 NCB - 1.
// Q4: the matrix is in Q4NX order (wstream.h): W = bf16_rne(q s + min') with a (scale, min') word per K-step of a cell
// (32 rows) instead of one (scale, zero point) word per group; a block carries 4 KiB of such words, KiB t for K-step t,
// and the operand of K-step t is dequantised with its own word.  Same loop otherwise: four scale-word requests per
// tile and group instead of one, two more instructions per operand (the word's halves to two fp32 registers) instead
// of three per group.
template <int NCB, bool Q4>
__device__ __forceinline__ void pf_tile(const PfArgs &p, unsigned char *lds, int m0, int col0) {
    constexpr int RT = kPfRowTiles, TM = kPfRows, WN = 16 * NCB, TN = 4 * WN;
    constexpr int kStageBytes = TM * 256;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    const int M = p.M, K = p.K, N = p.N, G = p.G;
    const int n0 = col0 + wave * WN;

    // x tile copy: instruction i of wave w fills rows 4 (16 w + i) .. + 3 of the stage.  Four consecutive instructions
    // share one LDS base (M0) and differ in the instruction's immediate offset, which the hardware adds to the LDS
    // address and to the global address alike; the global side takes it back through the scalar base.  (44 fewer
    // instructions per two groups than one M0 value per request; the run time did not move, 202 us either way: with
    // 1045 other instructions against 1024 free slots the loop is no longer bound by instruction issue.)
    const int c_row = lane >> 4, c_slot = lane & 15;
    uint32_t a_voff[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        int row = 4 * (16 * wave + i) + c_row;
        const int chunk = c_slot ^ (row & 15);
        if (m0 + row >= M) row = M - 1 - m0;   // ragged M: copy a row in range, never stored
        a_voff[i] = (uint32_t)((size_t)row * K * sizeof(uint16_t) + chunk * 16);
    }
    const char *a_base = reinterpret_cast<const char *>(p.x + (size_t)m0 * K);
    // request i (of 16) of the x tile copy of one group; src = this workgroup's rows at the group's 128 columns
    auto touch_voff = [&]() {
        asm volatile("" : "+v"(a_voff[0]), "+v"(a_voff[1]), "+v"(a_voff[2]), "+v"(a_voff[3]), "+v"(a_voff[4]), "+v"(a_voff[5]), "+v"(a_voff[6]), "+v"(a_voff[7]));
        asm volatile("" : "+v"(a_voff[8]), "+v"(a_voff[9]), "+v"(a_voff[10]), "+v"(a_voff[11]), "+v"(a_voff[12]), "+v"(a_voff[13]), "+v"(a_voff[14]), "+v"(a_voff[15]));
    };
    struct XSrc {
        gptr q[4];   // the group's source address minus 0, 1, 2, 3 KiB
    };
    auto copy_x_part = [&](int stage, const XSrc &src, int i) {
        auto *dst = (__attribute__((address_space(3))) void *)(lds + stage * kStageBytes + (16 * wave + (i & ~3)) * 1024);
        switch (i & 3) {
            case 0: __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src.q[0] + a_voff[i]), dst, 16, 0, 0); break;
            case 1: __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src.q[1] + a_voff[i]), dst, 16, 1024, 0); break;
            case 2: __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src.q[2] + a_voff[i]), dst, 16, 2048, 0); break;
            default: __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src.q[3] + a_voff[i]), dst, 16, 3072, 0); break;
        }
    };
    auto x_src = [&](int g) {
        const gptr b = scalar_ptr(a_base + (size_t)g * 256);
        return XSrc{{b, scalar_sub(b, 1024), scalar_sub(b, 2048), scalar_sub(b, 3072)}};
    };

    // this wave's NCB tiles of the stream-order buffer
    constexpr int MDK = Q4 ? kWsQ4MdKiB : 1;   // KiB of scale words in front of a block's cells, words per (group, column)
    const size_t tile_bytes = (size_t)(MDK * p.NB + G) * kWsCellBytes;
    const bool pair = p.epi == kEpiSwigluPair;
    const char *wt = p.w + (size_t)((pair ? n0 / 2 : n0) / kWsTileCols) * tile_bytes;
    u32x4 cell[2][NCB];
    uint32_t md[2][NCB][MDK];
    uint32_t lane16 = (uint32_t)lane * 16, ln16 = (uint32_t)ln * 16;
    // Scale word and cell of tile c for group g: lane 16 (gl / 4) + ln, dword gl % 4 of the block's first KiB, and the
    // (1 + gl)-th KiB of the block.  The tiles' base addresses stay in scalar registers and the group's offset is
    // folded into two per-lane offsets once per group (w_offsets), so that a tile costs its two requests and nothing
    // else in the loop.
    gptr tile_base[NCB];
#pragma unroll
    for (int c = 0; c < NCB; ++c) {
        const char *t = wt + (size_t)c * tile_bytes;
        if (pair && NCB % 2 == 0)   // tiles NCB / 2 .. NCB - 1 of the wave: the same columns of the second matrix
            t = c < NCB / 2 ? t : p.w_up + (t - p.w) - (size_t)(NCB / 2) * tile_bytes;
        tile_base[c] = scalar_ptr(t);
    }
    struct WOffsets {
        uint32_t md, cell;
    };
    auto w_offsets = [&](int g) {
        const int gl = g & 15;
        const uint32_t blk = (uint32_t)(g >> 4) * (uint32_t)((kWsBlockGroups + MDK) * kWsCellBytes);
        WOffsets o{ln16 + (blk + 256 * (gl >> 2) + 4 * (gl & 3)), lane16 + (blk + (uint32_t)(MDK + gl) * (uint32_t)kWsCellBytes)};
        asm volatile("" : "+v"(o.md), "+v"(o.cell));
        return o;
    };
    auto load_w_tile = [&](int set, const WOffsets &o, int c) {
#pragma unroll
        for (int t = 0; t < MDK; ++t)   // (Q4NX order: the word of K-step t is 1 KiB further on, an immediate offset)
            md[set][c][t] = *reinterpret_cast<const __attribute__((address_space(1))) uint32_t *>(tile_base[c] + o.md + t * 1024);
        // (a plain load: the workgroups of the same band and column tile on this XCD read the same cells out of its L2)
        cell[set][c] = *reinterpret_cast<const __attribute__((address_space(1))) u32x4 *>(tile_base[c] + o.cell);
    };
    // The compiler does not see the explicit s_waitcnt below: with loads in flight it would wait for vmcnt(0) at the
    // first use of a register loaded a group earlier, i.e. right behind the requests for the next group, and expose
    // their whole latency.  Taking the registers over right behind the explicit wait puts the compiler's wait where
    // the counter is already zero.
    auto take_w = [&](int set) {
#pragma unroll
        for (int c = 0; c < NCB; ++c) {
#pragma unroll
            for (int t = 0; t < MDK; ++t) asm volatile("" : "+v"(md[set][c][t]));
#pragma unroll
            for (int t = 0; t < 4; ++t) asm volatile("" : "+v"(cell[set][c][t]));
        }
    };

    floatx4 acc[RT][NCB];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int c = 0; c < NCB; ++c) acc[r][c] = floatx4{0.f, 0.f, 0.f, 0.f};

    // per-lane LDS byte offsets of the A operand of row tile 0
    // of each (stage, K-step); the row tile is the instruction's offset field
    uint32_t a_addr[2][4];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            a_addr[st][t] = (uint32_t)(st * kStageBytes + ln * 256 + (((4 * t + lg) ^ ln) << 4));
            asm volatile("" : "+v"(a_addr[st][t]));   // kept in a register: recomputing it costs issue slots in the loop
        }
    auto read_a = [&](int stage, int t, int r) {
        return *reinterpret_cast<const bf16x8 *>(lds + a_addr[stage][t] + r * 4096);
    };

    // State carried from group to group: the A operands of K-step 0, the first B operand, the decoded scale words.
    // The A operands are double buffered: K-step t multiplies from a[t % 2] while a[(t + 1) % 2] is refilled.
    bf16x8 a[2][RT];
    bf16x8 b_cur;
    float sf[NCB], c0[NCB];

    // One quantisation group, software-pipelined over (K-step t, tile c, quarter of the 16 row tiles).  Behind every
    // MFMA of quarters 0..2 sits a slot of the next operand's dequant; those MFMAs have no issue slot to spare.  The
    // memory requests are spread over the group, between the quarters and behind the MFMAs of quarter 3 (two free
    // slots each): issued as a burst at the top of the group they leave the wave in the request queue with no MFMA
    // in flight (a third of the run time), and the four waves asking for their 16 A operands at once want twice what
    // the LDS delivers.
    //   - every K-step: the 16 LDS reads that fetch the A operands of the next K-step (K-step 3: of the next group's
    //     K-step 0, from the other stage);
    //   - K-steps 0 and 1: the 16 requests of the next group's x tile copy (in K-steps 1 and 2 the last of them is a
    //     few hundred cycles old when K-step 3 waits for it: 213 us instead of 203 us); K-step 0: its cells and scale
    //     words.
    // Before K-step 3 everything has landed and every LDS read of this stage has returned (s_waitcnt vmcnt(0)
    // lgkmcnt(0): K-step 3's operands are fetched during K-step 2), then the barrier: the other stage is complete and
    // this one may be overwritten from K-step 0 of the next group on.  (Waiting for the LDS reads there costs nothing
    // measurable: 208.9 against 208.1 us over three alternations.)
    // The last tile dequantises the next group's first operand, so the groups follow each other without a bubble.
    //
    // The last group requests its own data once more and prepares a "next group" nobody uses: one copy of the code
    // for all groups matters, because the accumulators must stay in the same AGPRs from the first MFMA to the last,
    // and in a second copy of the loop body the register allocator moves them, through VGPRs, right behind MFMAs it
    // does not know of.
    auto group_step = [&](int g, int stage, int set) {
        const int gn = g + 1 < G ? g + 1 : g;
        const XSrc xs = x_src(gn);
        // The zero extension of a lane offset must sit in the same basic block as its request to fold into the
        // instruction's 32-bit offset; taken opaque here, once per group, not next to the request (the compiler puts an
        // s_nop between an asm statement and an instruction that reads its output).
        touch_voff();
        const WOffsets wo = w_offsets(gn);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t == 3) {
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                take_w(set ^ 1);
            }
#pragma unroll
            for (int c = 0; c < NCB; ++c) {
                const bool last = t == 3 && c == NCB - 1;
                const int cn = c + 1 < NCB ? c + 1 : 0, tn = c + 1 < NCB ? t : (t + 1) & 3;
                DequantSlots dq;
                dq.w = last ? cell[set ^ 1][0][0] : cell[set][cn][tn];
                if constexpr (Q4) {
                    decode_md_q4(last ? md[set ^ 1][0][0] : md[set][cn][tn], dq.sf, dq.c0);
                } else {
                    if (last) decode_md(md[set ^ 1][0][0], sf[0], c0[0]);
                    dq.sf = sf[cn];
                    dq.c0 = c0[cn];
                }
                const bf16x8(&ac)[RT] = a[t & 1];
                // This tile's share of the LDS reads that fetch the next K-step's A operands: operands n0 .. n1 - 1, all of
                // them issued by the last tile but one, so that one wait at the head of the next K-step (instead of one
                // in front of every quarter, each an issue slot) finds them all arrived.  The first three go between
                // the quarters, where the compiler would otherwise put an s_nop (it separates asm statements that hand
                // a register on), the rest behind the MFMAs of quarter 3.
                constexpr int kReadTiles = NCB > 1 ? NCB - 1 : 1;   // (one tile per K-step: the reads share it)
                constexpr int kPerTile = (RT + kReadTiles - 1) / kReadTiles;
                const int n0 = c < kReadTiles ? c * RT / kReadTiles : RT, n1 = c < kReadTiles ? (c + 1) * RT / kReadTiles : RT;
                if (c == 0) {   // two statements: an asm statement takes 30 operands at most
                    bf16x8(&an)[RT] = a[t & 1];
                    asm volatile("" : "+v"(an[0]), "+v"(an[1]), "+v"(an[2]), "+v"(an[3]), "+v"(an[4]), "+v"(an[5]), "+v"(an[6]), "+v"(an[7]));
                    asm volatile("" : "+v"(an[8]), "+v"(an[9]), "+v"(an[10]), "+v"(an[11]), "+v"(an[12]), "+v"(an[13]), "+v"(an[14]), "+v"(an[15]));
                }
                auto fetch_a = [&](int n) {
                    if (n < n1) a[(t + 1) & 1][n] = t < 3 ? read_a(stage, t + 1, n) : read_a(stage ^ 1, 0, n);
                };
                __builtin_amdgcn_sched_barrier(0);
                mfma_quarter<0>(acc[0][c], acc[1][c], acc[2][c], acc[3][c], ac[0], ac[1], ac[2], ac[3], b_cur, dq);
                __builtin_amdgcn_sched_barrier(0);
                fetch_a(n0);
                __builtin_amdgcn_sched_barrier(0);
                mfma_quarter<1>(acc[4][c], acc[5][c], acc[6][c], acc[7][c], ac[4], ac[5], ac[6], ac[7], b_cur, dq);
                __builtin_amdgcn_sched_barrier(0);
                fetch_a(n0 + 1);
                __builtin_amdgcn_sched_barrier(0);
                mfma_quarter<2>(acc[8][c], acc[9][c], acc[10][c], acc[11][c], ac[8], ac[9], ac[10], ac[11], b_cur, dq);
                __builtin_amdgcn_sched_barrier(0);
                fetch_a(n0 + 2);
                // quarter 3: the dequant is done, two issue slots are free behind each MFMA: the other requests
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    __builtin_amdgcn_sched_barrier(0);
                    mfma_one(acc[12 + k][c], ac[12 + k], b_cur);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int n = n0 + 3 + k * (kPerTile - 3) / 4; n < n0 + 3 + (k + 1) * (kPerTile - 3) / 4; ++n) fetch_a(n);
                    // the next group's x tile (K-steps 0 and 1: early enough to have landed before K-step 3) ...
                    if (t == 0 || t == 1) {
                        const int j = (t * NCB + c) * 4 + k;
#pragma unroll
                        for (int n = j * RT / (8 * NCB); n < (j + 1) * RT / (8 * NCB); ++n) copy_x_part(stage ^ 1, xs, n);
                    }
                    // ... its cells and scale words (K-step 0) ...
                    if (t == 0 && k == 3) load_w_tile(set ^ 1, wo, c);
                    // ... and the scale words of its other tiles, behind the last MFMA of the group
                    if (!Q4 && last && k == 3) {
#pragma unroll
                        for (int n = 1; n < NCB; ++n) decode_md(md[set ^ 1][n][0], sf[n], c0[n]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                b_cur = dq.operand();
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int i = 0; i < RT; ++i) copy_x_part(0, x_src(0), i);   // (64-bit addresses here: once per tile)
#pragma unroll
    for (int c = 0; c < NCB; ++c) load_w_tile(0, w_offsets(0), c);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the x tile copy writes LDS behind the compiler's back
    __syncthreads();
    take_w(0);
    if constexpr (Q4) {
        decode_md_q4(md[0][0][0], sf[0], c0[0]);
    } else {
#pragma unroll
        for (int c = 0; c < NCB; ++c) decode_md(md[0][c][0], sf[c], c0[c]);
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) a[0][r] = read_a(0, 0, r);
    b_cur = dequant_operand(cell[0][0][0], sf[0], c0[0]);

    // two groups per trip (G is even): stage / register set 0, then 1
    for (int g = 0; g < G; g += 2) {
        group_step(g, 0, 0);
        group_step(g + 1, 1, 1);
    }

    // The bf16 tile leaves through LDS (the K loop is done with it): a lane holds 4 rows of one column, so stores
    // straight from the registers would be 2-byte stores in 32-byte runs; rows padded by 16 bytes, read back as
    // 16-byte chunks so that a wave instruction stores whole rows.
    constexpr int LDC = TN + 8;   // bf16 elements per padded row
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written their accumulators
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int c = 0; c < NCB; ++c) asm volatile("" : "+a"(acc[r][c]));   // and no read of them moves above that wait
    __syncthreads();                                      // every wave is done reading the last x tile
    uint16_t *ct = reinterpret_cast<uint16_t *>(lds);
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int c = 0; c < NCB; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                ct[(16 * r + 4 * lg + i) * LDC + wave * WN + 16 * c + ln] = float_to_bf16_bits(acc[r][c][i]);
    __syncthreads();
    constexpr int CPR = TN / 8;   // 16-byte chunks per row
    // Epilogues on the bf16 tile (the same four as the checkpoint-layout kernel's): plain store; residual add of the
    // bf16 product, y = bf16(bf16(x . W) + aux); SwiGLU with aux = the gate projection, y = bf16(silu(aux) * bf16(x . W)),
    // silu(g) = g / (1 + exp(-g)) in fp32; half-split RoPE of the bf16 product on columns [0, rope_cols), whose
    // partner chunk is in the same tile (the tile widths offered to such a launch are whole numbers of heads).
    auto store_tile = [&](auto EPI) {
        constexpr int kEpi = decltype(EPI)::value;
        for (int chunk = threadIdx.x; chunk < TM * CPR; chunk += kPfThreads) {
            const int row = chunk / CPR, cc = chunk % CPR;
            if (m0 + row >= M) continue;
            u32x4 v = *reinterpret_cast<const u32x4 *>(&ct[row * LDC + 8 * cc]);
            const int grow = m0 + row, gcol = col0 + 8 * cc;
            const size_t at = (size_t)grow * N + gcol;
            if constexpr (kEpi == kEpiRope) {
                if (gcol < p.rope_cols) {
                    const int hd = p.rope_hd, half = hd >> 1;
                    const int i = gcol & (hd - 1);
                    const bool low = i < half;
                    const u32x4 w2 = *reinterpret_cast<const u32x4 *>(&ct[row * LDC + 8 * cc + (low ? half : -half)]);
                    const uint16_t *lut = p.aux + (size_t)(p.rope_pos0 + grow) * hd + (low ? i : i - half);
                    const u32x4 cs = *reinterpret_cast<const u32x4 *>(lut), sn = *reinterpret_cast<const u32x4 *>(lut + half);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t vw = v[e], ww = w2[e], cw = cs[e], sw = sn[e];
                        const float x0 = bf16_bits_to_float(vw & 0xFFFFu), x1 = bf16_bits_to_float(vw >> 16);
                        const float y0 = bf16_bits_to_float(ww & 0xFFFFu), y1 = bf16_bits_to_float(ww >> 16);
                        const float c0 = bf16_bits_to_float(cw & 0xFFFFu), c1 = bf16_bits_to_float(cw >> 16);
                        const float s0 = bf16_bits_to_float(sw & 0xFFFFu), s1 = bf16_bits_to_float(sw >> 16);
                        v[e] = low ? pack_bf16x2(x0 * c0 - y0 * s0, x1 * c1 - y1 * s1)
                                   : pack_bf16x2(x0 * c0 + y0 * s0, x1 * c1 + y1 * s1);
                    }
                }
            } else if constexpr (kEpi != kEpiNone) {
                const u32x4 a4 = *reinterpret_cast<const u32x4 *>(p.aux + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t vw = v[e], aw = a4[e];
                    const float v0 = bf16_bits_to_float(vw & 0xFFFFu), v1 = bf16_bits_to_float(vw >> 16);
                    const float a0 = bf16_bits_to_float(aw & 0xFFFFu), a1 = bf16_bits_to_float(aw >> 16);
                    if constexpr (kEpi == kEpiAddRounded) v[e] = pack_bf16x2(v0 + a0, v1 + a1);
                    else v[e] = pack_bf16x2(a0 / (1.0f + expf(-a0)) * v0, a1 / (1.0f + expf(-a1)) * v1);
                }
            }
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p.y + at));   // y is not read again here: keep x and W in L2
        }
    };
    if (pair) {
        if constexpr (NCB % 2 == 0) {
            constexpr int HW = WN / 2, OCPR = TN / 16;   // output columns per wave, 16-byte output chunks per row
            const int Nout = N, ocol0 = col0 / 2;
            for (int chunk = threadIdx.x; chunk < TM * OCPR; chunk += kPfThreads) {
                const int row = chunk / OCPR, oc = 8 * (chunk % OCPR);
                if (m0 + row >= M) continue;
                const uint16_t *src = &ct[row * LDC + (oc / HW) * WN + oc % HW];
                const u32x4 gv = *reinterpret_cast<const u32x4 *>(src), uv = *reinterpret_cast<const u32x4 *>(src + HW);
                u32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float g0 = bf16_bits_to_float(gv[e] & 0xFFFFu), g1 = bf16_bits_to_float(gv[e] >> 16);
                    const float u0 = bf16_bits_to_float(uv[e] & 0xFFFFu), u1 = bf16_bits_to_float(uv[e] >> 16);
                    v[e] = pack_bf16x2(g0 / (1.0f + expf(-g0)) * u0, g1 / (1.0f + expf(-g1)) * u1);
                }
                *reinterpret_cast<u32x4 *>(p.y + (size_t)(m0 + row) * Nout + ocol0 + oc) = v;
            }
        }
    } else if (p.epi == kEpiAddRounded) store_tile(std::integral_constant<int, kEpiAddRounded>{});
    else if (p.epi == kEpiSiluGateMul) store_tile(std::integral_constant<int, kEpiSiluGateMul>{});
    else if (p.epi == kEpiRope) store_tile(std::integral_constant<int, kEpiRope>{});
    else store_tile(std::integral_constant<int, kEpiNone>{});
}

// Tile order of one width: the row panels are cut into bands of `band` panels; inside a band the order runs down the
// band's panels first, then to the next column tile.  An XCD takes a contiguous range of that order, so the
// workgroups that run together on it cover band x (32 / band) tiles: they share `band` x panels and 32 / band weight
// slabs in its L2, and over the launch a weight slab is fetched by tiles_m / band XCDs instead of by every one.
__device__ __forceinline__ void pf_tile_of(int idx, int tiles_m, int n_cols, int band, int &row, int &col) {
    const int per_band = band * n_cols, b = idx / per_band, r = idx - b * per_band;
    const int rows = min(band, tiles_m - b * band);   // (the last band may be short)
    row = b * band + r % rows;
    col = r / rows;
}

// blockIdx -> tile.  The wide tiles come first in dispatch order, so that the narrow ones fill in behind them.  Each
// XCD (blockIdx % 8) takes a contiguous range of the tiles of either width in the order of pf_tile_of.
template <int NW, int NN, bool Q4>
__global__ void __launch_bounds__(kPfThreads, 1) gemm_wsp_kernel(const PfArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int wide_total = p.tiles_m * p.n_wide, narrow_total = p.tiles_m * p.n_narrow;
    const int wide_per_xcd = (wide_total + 7) / 8, narrow_per_xcd = (narrow_total + 7) / 8;
    if (slot < wide_per_xcd) {
        const int tile = xcd * wide_per_xcd + slot;
        if (tile >= wide_total) return;
        int row, col;
        pf_tile_of(tile, p.tiles_m, p.n_wide, p.band, row, col);
        pf_tile<NW, Q4>(p, lds, row * kPfRows, col * 64 * NW);
    } else if constexpr (NN > 0) {
        const int tile = xcd * narrow_per_xcd + (slot - wide_per_xcd);
        if (tile >= narrow_total) return;
        int row, col;
        pf_tile_of(tile, p.tiles_m, p.n_narrow, p.band, row, col);
        pf_tile<NN, Q4>(p, lds, row * kPfRows, p.n_wide * 64 * NW + col * 64 * NN);
    }
}

// Column tiling of N = 64 U columns.  Normally a tiles of 256 and b tiles of 192 (4 a + 3 b = U): the split that
// finishes first when tiles_m * (a + b) tiles are handed, wide ones first, to `cus` CUs as they fall free (tile time
// taken as proportional to its width).  A matrix with too few such tiles for the chip (N = 2048, M = 2048: 64) is cut
// into tiles of 128 or 64 columns instead: those read the x tile from LDS two and four times as often per MFMA (the
// LDS delivers half of what the 64-column tile asks for), which is still better than idle CUs.
struct Widths {
    int ncb;            // columns / 64 of the "wide" tiles: 4, or 2 / 1 for the narrow uniform tilings
    int wide, narrow;   // number of column tiles of ncb * 64 columns and of the narrow width
    int ncb_narrow = 3; // columns / 64 of the narrow tiles of a mixed launch: 3, or 2 where tiles must be halves or whole heads
};

double split_cost(long n_wide_tiles, long n_narrow_tiles, int cus, double narrow_cost) {
    // greedy list scheduling of two task sizes, big first, on identical machines: the finishing times after the
    // wide tiles are 4 q (+ 4 on r machines); every narrow tile goes to the machine that falls free first
    std::vector<double> load(cus);
    const long q = n_wide_tiles / cus, r = n_wide_tiles % cus;
    for (int i = 0; i < cus; ++i) load[i] = 4.0 * (q + (i < r ? 1 : 0));
    std::make_heap(load.begin(), load.end(), std::greater<double>());
    for (long i = 0; i < n_narrow_tiles; ++i) {
        std::pop_heap(load.begin(), load.end(), std::greater<double>());
        load.back() += narrow_cost;
        std::push_heap(load.begin(), load.end(), std::greater<double>());
    }
    return *std::max_element(load.begin(), load.end());
}

// `heads128`: every tile must hold whole heads of 128 columns (RoPE epilogue) or halve into whole 16-column tiles
// (gate and up in one tile): no 192- or 64-column tiles; the wide tiles are then mixed with 128-column ones.
Widths pick_widths(int tiles_m, int U, int cus, bool heads128) {
    struct Entry {
        int tiles_m, U, cus;
        bool heads128;
        Widths w;
    };
    static std::mutex mu;
    static Entry cache[8] = {};
    static int next = 0;
    std::lock_guard<std::mutex> lock(mu);
    for (const Entry &e : cache)
        if (e.U == U && e.tiles_m == tiles_m && e.cus == cus && e.heads128 == heads128) return e.w;
    Widths best{4, -1, -1};
    double best_cost = -1;
    const int nn = heads128 ? 2 : 3;
    const double narrow_cost = heads128 ? 2 * kPfSlowdown128 : 3.0;
    for (int a = U / 4; a >= 0; --a) {   // ties go to the split with more wide tiles
        if ((U - 4 * a) % nn) continue;
        const int b = (U - 4 * a) / nn;
        if (a == 0 && heads128) continue;   // (the uniform 128-column tiling is priced below)
        const double cost = split_cost((long)tiles_m * a, (long)tiles_m * b, cus, narrow_cost);
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = Widths{4, a, b, nn};
        }
    }
    // uniform narrow tilings: rounds x width x (measured) slowdown of the narrower tile's inner loop
    const struct { int ncb; double slowdown; } narrow[2] = {{2, kPfSlowdown128}, {1, kPfSlowdown64}};
    for (const auto &nv : narrow) {
        if (U % nv.ncb || (heads128 && nv.ncb == 1)) continue;
        const long tiles = (long)tiles_m * (U / nv.ncb);
        const double cost = (double)((tiles + cus - 1) / cus) * nv.ncb * nv.slowdown;
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = Widths{nv.ncb, U / nv.ncb, 0, 3};
        }
    }
    cache[next] = Entry{tiles_m, U, cus, heads128, best};
    next = (next + 1) % 8;
    return best;
}

// Row panels per band.  Fetch traffic of a launch over 8 XCDs is about (tiles_m / band) x the weights + 2 band x the
// activations (a wide and a narrow pass): least at band 2 to 4 for M = 2048, N = 14336.  Measured there (us per launch,
// two boxes): band 1 205 / -, 2 198 / 192, 4 194 / 191, 8 196 / -; with plain instead of non-temporal cell loads and
// non-temporal stores of y on top: band 2 182, band 4 183 - 187.
int pf_band(int tiles_m) {
    const int want = g_gemv_ws_tune.prefill_band ? g_gemv_ws_tune.prefill_band : 2;
    return want < tiles_m ? want : tiles_m;
}

template <int NW, int NN, bool Q4>
hipError_t launch_wsp_q(const PfArgs &p, hipStream_t stream) {
    constexpr size_t kStages = 2 * (size_t)kPfRows * 256, kOut = (size_t)kPfRows * (64 * NW + 8) * sizeof(uint16_t);
    constexpr size_t kLds = kStages > kOut ? kStages : kOut;
    static_assert(kLds <= 160 * 1024, "tile does not fit LDS");
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_wsp_kernel<NW, NN, Q4>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds);
    if (e != hipSuccess) return e;
    const int wide_per_xcd = (p.tiles_m * p.n_wide + 7) / 8, narrow_per_xcd = (p.tiles_m * p.n_narrow + 7) / 8;
    const int grid = 8 * (wide_per_xcd + narrow_per_xcd);
    hipLaunchKernelGGL((gemm_wsp_kernel<NW, NN, Q4>), dim3(grid), dim3(kPfThreads), kLds, stream, p);
    return hipGetLastError();
}

template <int NW, int NN>
hipError_t launch_wsp(const PfArgs &p, hipStream_t stream) {
    return p.q4 ? launch_wsp_q<NW, NN, true>(p, stream) : launch_wsp_q<NW, NN, false>(p, stream);
}

}  // namespace

bool gemm_prefill_ws_supported(int M, int K, int N) { return M > 0 && K > 0 && K % (2 * kGroup) == 0 && N > 0 && N % 64 == 0; }

hipError_t launch_gemm_prefill_ws(const uint16_t *x, const void *w, uint16_t *y, int M, int K, int N, hipStream_t stream, int epi,
                                  const uint16_t *aux, const GemmRope *rope, bool q4) {
    if (!gemm_prefill_ws_supported(M, K, N)) return hipErrorInvalidValue;
    if ((epi != kEpiNone && !aux) || (epi == kEpiRope && (!rope || (rope->head_dim != 64 && rope->head_dim != 128) ||
                                                          rope->cols % rope->head_dim || N % rope->head_dim)))
        return hipErrorInvalidValue;
    PfArgs p{};
    p.x = x;
    p.w = static_cast<const char *>(w);
    p.y = y;
    p.aux = aux;
    p.epi = epi;
    p.q4 = q4;
    if (epi == kEpiRope) p.rope_cols = rope->cols, p.rope_hd = rope->head_dim, p.rope_pos0 = rope->pos0;
    const bool heads128 = epi == kEpiRope && rope->head_dim == 128;
    p.M = M, p.K = K, p.N = N, p.G = K / kGroup, p.NB = ws_blocks(K);
    p.tiles_m = (M + kPfRows - 1) / kPfRows;
    p.band = pf_band(p.tiles_m);
    const int U = N / 64;
    Widths wd = pick_widths(p.tiles_m, U, 256, heads128);
    // tuning: one tile width only (1: 256 columns, 2: 192, 3: 128, 4: 64) where it divides N; 5: 256 mixed with 128
    // where the launch takes that mix (RoPE heads of 128, gate and up in one tile)
    const int force = g_gemv_ws_tune.prefill_tile;
    if (force == 1 && U % 4 == 0) wd = Widths{4, U / 4, 0};
    if (force == 2 && U % 3 == 0 && !heads128) wd = Widths{4, 0, U / 3};
    if (force == 3 && U % 2 == 0) wd = Widths{2, U / 2, 0};
    if (force == 4 && !heads128) wd = Widths{1, U, 0};
    if (force == 5 && heads128 && U % 2 == 0 && U >= 6) wd = Widths{4, (U - 2) / 4, U % 4 == 0 ? 2 : 1, 2};
    p.n_wide = wd.wide, p.n_narrow = wd.narrow;
    if (wd.ncb == 2) return launch_wsp<2, 0>(p, stream);
    if (wd.ncb == 1) return launch_wsp<1, 0>(p, stream);
    if (wd.wide == 0) {
        p.n_wide = wd.narrow, p.n_narrow = 0;
        return launch_wsp<3, 0>(p, stream);
    }
    if (wd.narrow == 0) return launch_wsp<4, 0>(p, stream);
    return wd.ncb_narrow == 2 ? launch_wsp<4, 2>(p, stream) : launch_wsp<4, 3>(p, stream);
}

// h[M, H] = bf16(silu(bf16(x . W_gate)) * bf16(x . W_up)): both projections in one launch, a tile holding the same
// 128 (or 64) columns of either; the gate projection never leaves the chip.  H % 64 == 0.
hipError_t launch_gemm_prefill_ws_swiglu(const uint16_t *x, const void *w_gate, const void *w_up, uint16_t *h, int M, int K, int H,
                                         hipStream_t stream, bool q4) {
    if (!gemm_prefill_ws_supported(M, K, H) || !w_up) return hipErrorInvalidValue;
    PfArgs p{};
    p.x = x;
    p.w = static_cast<const char *>(w_gate);
    p.w_up = static_cast<const char *>(w_up);
    p.y = h;
    p.epi = kEpiSwigluPair;
    p.q4 = q4;
    p.M = M, p.K = K, p.N = H, p.G = K / kGroup, p.NB = ws_blocks(K);
    p.tiles_m = (M + kPfRows - 1) / kPfRows;
    p.band = pf_band(p.tiles_m);
    const int U = 2 * H / 64;   // the tile grid runs over 2 H columns; 192- and 64-column tiles cannot be halved
    Widths wd = pick_widths(p.tiles_m, U, 256, true);
    const int force = g_gemv_ws_tune.prefill_tile;
    if (force == 1 && U % 4 == 0) wd = Widths{4, U / 4, 0};
    if (force == 3) wd = Widths{2, U / 2, 0};
    if (force == 5 && U >= 6) wd = Widths{4, (U - 2) / 4, U % 4 == 0 ? 2 : 1, 2};
    p.n_wide = wd.wide, p.n_narrow = wd.ncb == 4 ? wd.narrow : 0;
    if (wd.ncb == 2) return launch_wsp<2, 0>(p, stream);
    return p.n_narrow ? launch_wsp<4, 2>(p, stream) : launch_wsp<4, 0>(p, stream);
}

}  // namespace w4a16
