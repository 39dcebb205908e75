// Prefill W4A16 GEMM for gfx950: y[M, N] = bf16(x[M, K] . W), M > 16.
//
// Compute-bound.  A workgroup (4 waves) owns a 256 x 256 output tile and walks K in steps of
// 64; each wave owns 128 x 128 of it as 4 x 4 v_mfma_f32_32x32x16_bf16 tiles (256 fp32
// accumulators per lane, one wave per SIMD).  Per K step the x tile is copied to LDS and the
// packed weight tile is dequantised ONCE per workgroup to bf16 - the same values the dense
// dequant produces, W = bf16_rne((q - z) * s) - and stored [n][k], so both MFMA operands are
// 16-byte LDS reads of 8 consecutive k.  LDS is double buffered (2 x 72 KiB of the 160 KiB):
// while the MFMAs run on one buffer the next tile is dequantised into the other, and the
// global loads for the tile after that are already in flight; one barrier per K step.
//
// LDS layout (checked with a ds_read_b128 / ds_write_b128 timing probe and SQ_LDS_BANK_CONFLICT;
// the LDS behaves as 64 banks of 4 B: a read pass is 16 lanes x 16 B, a write pass 8 lanes x 16 B).
// x tile: unpadded rows of 64 bf16 (128 B) filled by global_load_lds_dwordx4, 16-byte chunk c of
// row r at slot c ^ r % 8 (the lanes of a copy choose their global chunk accordingly), so the
// operand reads of 16 consecutive rows touch 16 distinct slots of a 256-byte window.
// Weight tile [n][k]: rows padded to 160 B and the chunk index XORed with (n / 8) % 8.  Reads
// (lanes = 16 consecutive n, same chunk): 160 n covers the even 16-byte slots of a 256-byte
// window for n = 0..7 and the XOR flips bit 0 for n = 8..15, which takes the odd slots.  Dequant
// stores (lanes = same column j of consecutive packed words, n = 8 * word + j): 1280 * word is
// 0 mod 128, so the slot is chunk ^ word % 8, distinct over 8 lanes; and the 8 columns of a lane
// are one base address plus j * 160 B.
//
// blockIdx -> tile: each XCD (blockIdx % 8) takes a contiguous range of tiles with N
// fastest, so one XCD's L2 keeps an x panel resident while the weight panels stream by.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int LDA = BK;                          // x tile rows are unpadded (128 B), chunks XOR-swizzled
constexpr int LDB = BK + 16;                     // padded LDS row of the weight tile (160 B), chunks XOR-swizzled
constexpr int kThreads = 256;
#ifndef VALU_SLOTS
#define VALU_SLOTS 5
#endif
constexpr int kStageElems = BM * LDA + BN * LDB; // bf16 elements per stage
constexpr size_t kLdsBytes = 2 * kStageElems * sizeof(uint16_t);

struct GemmParams {
    const uint16_t *x;
    const uint32_t *qw;
    const uint32_t *qz;
    const uint16_t *sc;
    uint16_t *y;
    const uint16_t *aux;   // [M, N] bf16 operand of the epilogue (residual or gate), or nullptr
    int epi;               // kEpi*
    int M, K, N;
    int tiles_m, tiles_n;
    int rope_cols, rope_hd, rope_pos0;   // kEpiRope: columns [0, rope_cols) are heads of rope_hd to rotate, row m is position rope_pos0 + m
    float *partial;        // split-K: fp32 [gridDim.y][M][N] partial products instead of y (nullptr: no split)
    int kt_per_split;      // K steps of 64 per blockIdx.y (even)
};

__global__ void __launch_bounds__(kThreads, 1) gemm_kernel(const GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    const int tm = tile / p.tiles_n, tn = tile % p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int nb = p.N >> 3;

    // ---- staging assignments ----
    // x tile: copied global -> LDS without passing through registers (global_load_lds_dwordx4).
    // One wave instruction fills 1 KiB of LDS linearly with lane l's 16 bytes at 16 * l, i.e. 8
    // rows of 128 B; lane l = (row l / 8, slot l % 8) fetches chunk slot ^ row % 8 of its row, so
    // that chunk c of row r sits at slot c ^ r % 8 (the operand reads of consecutive rows are then
    // conflict-free without padding).  Wave w, instruction i covers rows 32 i + 8 w .. + 7.
    const int a_slot = lane & 7, a_sub = lane >> 3;
    uint32_t a_voff[8];                             // byte offsets from x + m0 * K + k0
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int row = 32 * i + 8 * wave + a_sub;
        if (m0 + row >= p.M) row = p.M - 1 - m0;    // ragged M: load in range, never stored
        a_voff[i] = (uint32_t)(((size_t)row * p.K + 8 * (a_slot ^ a_sub)) * sizeof(uint16_t));
    }
    const char *a_base = reinterpret_cast<const char *>(p.x + (size_t)m0 * p.K);
    // weight tile: thread takes packed word column tid % 32 (8 columns) for the 8 rows of octet tid / 32.
    const int b_col = tid & 31, b_oct = tid >> 5;
    int b_word = (n0 >> 3) + b_col;
    if (b_word >= nb) b_word = nb - 1;              // ragged N
    const uint32_t b_voff = (uint32_t)(((size_t)(8 * b_oct) * nb + b_word - (n0 >> 3)) * sizeof(uint32_t));
    const char *b_base = reinterpret_cast<const char *>(p.qw + (n0 >> 3));
    const int b_chunk = b_oct ^ (b_col & 7);        // swizzled 16-byte chunk inside the LDS row: oct ^ (n / 8) % 8

    uint32_t rb[2][8];                              // two register sets: tiles kt + 1 and kt + 2
    float zs[8], sf[8];                             // -z * s and s of this thread's 8 columns

    auto dma_a = [&](uint16_t *st, int k0) {
        const char *src = a_base + (size_t)k0 * sizeof(uint16_t);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void *)(src + a_voff[i]),
                (__attribute__((address_space(3))) void *)(st + (32 * i + 8 * wave) * LDA), 16, 0, 0);
    };
    auto load_b = [&](int k0, uint32_t (&dst)[8]) {
        const char *src = b_base + (size_t)k0 * nb * sizeof(uint32_t);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            dst[i] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(src + (size_t)i * nb * sizeof(uint32_t) + b_voff));
    };
    uint32_t raw_z;
    u32x4 rs;
    auto fetch_group = [&](int k0) {                // issue the loads; convert_group() consumes them later
        const int g = k0 / kGroup;
        raw_z = p.qz[(size_t)g * nb + b_word];
        rs = *reinterpret_cast<const u32x4 *>(p.sc + (size_t)g * p.N + 8 * (size_t)b_word);
    };
    auto convert_group = [&]() {
        float z[8];
        unpack8_f32(raw_z, z);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sf[2 * j] = bf16_bits_to_float(rs[j] & 0xFFFFu);
            sf[2 * j + 1] = bf16_bits_to_float(rs[j] >> 16);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) zs[j] = -z[j] * sf[j];   // exact: 4 x 8 significant bits
    };
    // weight columns 2 * part, 2 * part + 1 (all 8 k of each) -> LDS.  q * s - z * s equals (q - z) * s exactly.
    auto store_b = [&](uint16_t *st, const uint32_t (&src)[8], int part) {
        uint16_t *sB = st + BM * LDA;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = 2 * part + h;              // natural column inside the packed word
            const int sh = 4 * unpack_pos(j);
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = fmaf(static_cast<float>((src[i] >> sh) & 0xFu), sf[j], zs[j]);
            u32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
            *reinterpret_cast<u32x4 *>(&sB[(8 * b_col + j) * LDB + 8 * b_chunk]) = o;
        }
    };

    floatx16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int fr = lane & 31;          // row (A) / column (B) inside a 32-wide MFMA tile
    const int fk = lane >> 5;          // which 8-k half of a 16-k MFMA step
    // per-lane LDS offsets of the operand fragments (elements), without the k term
    int a_off[4], b_off[4], b_sw[4];
    const int a_sw = fr & 7;
#pragma unroll
    for (int i = 0; i < 4; ++i) a_off[i] = (wm * 128 + i * 32 + fr) * LDA;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = wn * 128 + j * 32 + fr;
        b_off[j] = n * LDB;
        b_sw[j] = (n >> 3) & 7;
    }

    // K steps [kt_begin, kt_end) of this workgroup: all of them, or slice blockIdx.y of a split-K launch (even bounds)
    const int kt_begin = blockIdx.y * p.kt_per_split, kt_end = kt_begin + p.kt_per_split;
    uint16_t *stage0 = lds, *stage1 = lds + kStageElems;

    // Pipeline (stage = kt % 2, one barrier per K step).  While the MFMAs of tile kt run:
    //   - x of tile kt + 1 is loaded (L2-resident panel) at the top of the step and stored to
    //     the other stage in its last quarter;
    //   - the packed weights of tile kt + 1, loaded during the previous step, are dequantised
    //     into the other stage, a quarter per MFMA group;
    //   - the packed weights of tile kt + 2 are loaded into the other register set.
    // A step is one basic block (the flags are compile-time), and sched_group_barrier pins the
    // interleaving: one wave per SIMD issues in order, so VALU / LDS / global instructions only
    // overlap with the matrix pipe when they sit between MFMAs in program order.
    dma_a(stage0, kt_begin * BK);
    load_b(kt_begin * BK, rb[0]);
    fetch_group(kt_begin * BK);
    convert_group();
#pragma unroll
    for (int part = 0; part < 4; ++part) store_b(stage0, rb[0], part);
    load_b((kt_begin + 1) * BK, rb[1]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the x tile copy writes LDS behind the compiler's back
    __syncthreads();

    auto read_frags = [&](const uint16_t *st, int kk, bf16x8 (&a)[4], bf16x8 (&b)[4]) {
        const uint16_t *sA = st, *sB = st + BM * LDA;
        const int chunk = 2 * kk + fk;
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const bf16x8 *>(&sA[a_off[i] + 8 * (chunk ^ a_sw)]);
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const bf16x8 *>(&sB[b_off[j] + 8 * (chunk ^ b_sw[j])]);
    };

    // NEXT: tile kt + 1 exists; AFTER: tile kt + 2 exists; ODD: kt is odd.  With BK = 64 a new
    // quantisation group opens at every even tile: on odd kt tile kt + 1 opens one (convert the
    // registers fetched a step ago), on even kt tile kt + 2 does (fetch them now).
    auto step = [&](int kt, uint16_t *cur, uint16_t *nxt, uint32_t (&rb_next)[8], uint32_t (&rb_after)[8],
                    auto NEXT, auto AFTER, auto ODD) {
        bf16x8 fa[2][4], fb[2][4];
        // Everything that was loaded into registers earlier is taken over before the x tile copy is
        // issued: with a copy to LDS pending the compiler waits for vmcnt(0) at the first use of
        // any loaded register, which would expose the copy's latency in every step.
        uint32_t rbn[8];
        if (NEXT) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                rbn[i] = rb_next[i];
                asm volatile("" : "+v"(rbn[i]));
            }
            if (ODD) convert_group();
#pragma unroll
            for (int j = 0; j < 8; ++j) asm volatile("" : "+v"(zs[j]), "+v"(sf[j]));
            dma_a(nxt, (kt + 1) * BK);
        }
        if (AFTER) {
            load_b((kt + 2) * BK, rb_after);
            if (!ODD) fetch_group((kt + 2) * BK);
        }
        read_frags(cur, 0, fa[0], fb[0]);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            if (kk < 3) read_frags(cur, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
            if (NEXT) store_b(nxt, rbn, kk);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
            // 16 MFMAs, each followed by a slice of the other work of this quarter
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // DS read
                __builtin_amdgcn_sched_group_barrier(0x002, VALU_SLOTS, 0);   // VALU
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // DS write
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // VMEM read
            }
        }
        if (NEXT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // x tile copy of kt + 1 has landed in LDS
        __syncthreads();
    };
    using T = std::true_type;
    using F = std::false_type;
    int kt = kt_begin;
    for (; kt + 3 < kt_end; kt += 2) {
        step(kt, stage0, stage1, rb[1], rb[0], T{}, T{}, F{});
        step(kt + 1, stage1, stage0, rb[0], rb[1], T{}, T{}, T{});
    }
    // the step count is even: two steps remain
    step(kt, stage0, stage1, rb[1], rb[0], T{}, F{}, F{});
    step(kt + 1, stage1, stage0, rb[0], rb[1], F{}, F{}, T{});

    // D layout of the 32x32 MFMA: register r of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32:
    // a lane holds a column, so stores straight from the registers are 2-byte stores in 64-byte runs
    // (256 store instructions per thread, ~8 us per tile).  Instead the bf16 tile is transposed through
    // LDS, which the K loop no longer needs (its last step ended with a barrier): rows padded to 528 B
    // (the two row groups of a wave instruction, 4 rows apart, land 16 banks apart), then read back as
    // 16-byte chunks so that a wave stores two whole 512-byte rows per instruction and the epilogue
    // operand is loaded the same way.
    constexpr int LDC = BN + 8;
    static_assert((size_t)BM * LDC * sizeof(uint16_t) <= kLdsBytes, "the output tile must fit the K loop's LDS");
    auto store_tile = [&](auto EPI) {
        uint16_t *ct = lds;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    ct[(wm * 128 + i * 32 + 8 * (r >> 2) + 4 * fk + (r & 3)) * LDC + wn * 128 + j * 32 + fr] =
                        float_to_bf16_bits(acc[i][j][r]);
        __syncthreads();
#pragma unroll 4
        for (int k = 0; k < BM * BN / 8 / kThreads; ++k) {
            const int chunk = tid + kThreads * k;
            const int row = chunk >> 5, c = chunk & 31;           // 32 chunks of 8 columns per row
            const int grow = m0 + row, gcol = n0 + 8 * c;
            if (grow >= p.M || gcol >= p.N) continue;             // N % 8 == 0: a chunk is inside or outside
            u32x4 v = *reinterpret_cast<const u32x4 *>(&ct[row * LDC + 8 * c]);
            const size_t at = (size_t)grow * p.N + gcol;
            if constexpr (decltype(EPI)::value == kEpiRope) {
                // Half-split rotation of the bf16 product: out[i] = x[i] cos[i] - x[i + h] sin[i],
                // out[i + h] = x[i + h] cos[i] + x[i] sin[i]; the partner chunk is in the same tile
                // (a tile is a whole number of heads).  Products of two bf16 values are exact in fp32,
                // so each element is rounded once, fused multiply-add or not.
                if (gcol < p.rope_cols) {
                    const int hd = p.rope_hd, half = hd >> 1;
                    const int i = gcol & (hd - 1);
                    const bool low = i < half;
                    const u32x4 w = *reinterpret_cast<const u32x4 *>(&ct[row * LDC + 8 * c + (low ? half : -half)]);
                    const uint16_t *lut = p.aux + (size_t)(p.rope_pos0 + grow) * hd + (low ? i : i - half);
                    const u32x4 cs = *reinterpret_cast<const u32x4 *>(lut), sn = *reinterpret_cast<const u32x4 *>(lut + half);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t vw = v[e], ww = w[e], cw = cs[e], sw = sn[e];
                        const float x0 = bf16_bits_to_float(vw & 0xFFFFu), x1 = bf16_bits_to_float(vw >> 16);
                        const float y0 = bf16_bits_to_float(ww & 0xFFFFu), y1 = bf16_bits_to_float(ww >> 16);
                        const float c0 = bf16_bits_to_float(cw & 0xFFFFu), c1 = bf16_bits_to_float(cw >> 16);
                        const float s0 = bf16_bits_to_float(sw & 0xFFFFu), s1 = bf16_bits_to_float(sw >> 16);
                        v[e] = low ? pack_bf16x2(x0 * c0 - y0 * s0, x1 * c1 - y1 * s1)
                                   : pack_bf16x2(x0 * c0 + y0 * s0, x1 * c1 + y1 * s1);
                    }
                }
            } else if constexpr (decltype(EPI)::value != kEpiNone) {
                const u32x4 a = *reinterpret_cast<const u32x4 *>(p.aux + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t vw = v[e], aw = a[e];
                    const float v0 = bf16_bits_to_float(vw & 0xFFFFu), v1 = bf16_bits_to_float(vw >> 16);
                    const float a0 = bf16_bits_to_float(aw & 0xFFFFu), a1 = bf16_bits_to_float(aw >> 16);
                    if constexpr (decltype(EPI)::value == kEpiAddRounded) {
                        // y = bf16(bf16(x . W) + R): the product is a bf16 tensor before the add
                        v[e] = pack_bf16x2(v0 + a0, v1 + a1);
                    } else {
                        // y = bf16(silu(G) * bf16(x . W)), silu(g) = g / (1 + exp(-g)) in fp32
                        v[e] = pack_bf16x2(a0 / (1.0f + expf(-a0)) * v0, a1 / (1.0f + expf(-a1)) * v1);
                    }
                }
            }
            *reinterpret_cast<u32x4 *>(p.y + at) = v;
        }
    };
    if (p.partial) {
        float *dst = p.partial + (size_t)blockIdx.y * p.M * p.N;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = n0 + wn * 128 + j * 32 + fr;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * fk + (r & 3);
                    if (row < p.M && col < p.N) dst[(size_t)row * p.N + col] = acc[i][j][r];
                }
            }
    } else if (p.epi == kEpiAddRounded)
        store_tile(std::integral_constant<int, kEpiAddRounded>{});
    else if (p.epi == kEpiSiluGateMul)
        store_tile(std::integral_constant<int, kEpiSiluGateMul>{});
    else if (p.epi == kEpiRope)
        store_tile(std::integral_constant<int, kEpiRope>{});
    else
        store_tile(std::integral_constant<int, kEpiNone>{});
}

}  // namespace

// y = epilogue(sum over slices of the split-K partial products), four elements per thread.
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *__restrict__ partial, int ksplit, size_t mn,
                                                            uint16_t *__restrict__ y, const uint16_t *__restrict__ aux, int epi) {
    const size_t at = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (at >= mn) return;                            // M * N is a multiple of 4 (N % 32 == 0)
    floatx4 sum = *reinterpret_cast<const floatx4 *>(partial + at);
    for (int s = 1; s < ksplit; ++s) sum += *reinterpret_cast<const floatx4 *>(partial + (size_t)s * mn + at);
    uint16_t out[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        out[e] = float_to_bf16_bits(sum[e]);
        if (epi == kEpiAddRounded) {
            out[e] = float_to_bf16_bits(bf16_bits_to_float(out[e]) + bf16_bits_to_float(aux[at + e]));
        } else if (epi == kEpiSiluGateMul) {
            const float g = bf16_bits_to_float(aux[at + e]);
            out[e] = float_to_bf16_bits(g / (1.0f + expf(-g)) * bf16_bits_to_float(out[e]));
        }
    }
    *reinterpret_cast<uint2 *>(y + at) = uint2{(uint32_t)out[0] | ((uint32_t)out[1] << 16), (uint32_t)out[2] | ((uint32_t)out[3] << 16)};
}

// Slices along K for a launch whose tiles would leave most of the chip idle: as many as fit the CUs,
// at most 4, each an even number of K steps and at least 8 of them.
int gemm_prefill_ksplit(int M, int K, int N, int cus) {
    const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    const int KT = K / BK;
    int split = 1;
    for (int s = 2; s <= 4; s *= 2)
        if (tiles * s <= cus && KT % (2 * s) == 0 && KT / s >= 8) split = s;
    return split;
}

size_t gemm_prefill_splitk_bytes(int M, int K, int N, int cus) {
    const int s = gemm_prefill_ksplit(M, K, N, cus);
    return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

hipError_t launch_gemm_prefill(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                               const uint16_t *scales, uint16_t *y, int M, int K, int N, hipStream_t stream,
                               int epi, const uint16_t *aux, float *splitk_scratch, int cus, const GemmRope *rope) {
    // 144 KiB of dynamic LDS needs the attribute; it is per device, so it is set on every launch
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes);
    if (e != hipSuccess) return e;
    GemmParams p;
    p.x = x;
    p.qw = reinterpret_cast<const uint32_t *>(qweight);
    p.qz = reinterpret_cast<const uint32_t *>(qzeros);
    p.sc = scales;
    p.y = y;
    p.aux = aux;
    p.epi = aux ? epi : kEpiNone;
    p.rope_cols = rope ? rope->cols : 0;
    p.rope_hd = rope ? rope->head_dim : 64;
    p.rope_pos0 = rope ? rope->pos0 : 0;
    if (p.epi == kEpiRope && !rope) return hipErrorInvalidValue;
    p.M = M;
    p.K = K;
    p.N = N;
    p.tiles_m = (M + BM - 1) / BM;
    p.tiles_n = (N + BN - 1) / BN;
    // the reduction kernel of the split has no rotation epilogue
    const int ksplit = splitk_scratch && p.epi != kEpiRope ? gemm_prefill_ksplit(M, K, N, cus) : 1;
    p.partial = ksplit > 1 ? splitk_scratch : nullptr;
    p.kt_per_split = K / BK / ksplit;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(gemm_kernel, dim3(grid, ksplit), dim3(kThreads), kLdsBytes, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess || ksplit == 1) return e;
    const size_t mn = (size_t)M * N;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, stream, splitk_scratch,
                       ksplit, mn, y, p.aux, p.epi);
    return hipGetLastError();
}

}  // namespace w4a16
