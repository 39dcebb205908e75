// Split-K streaming W4A16 kernel for M <= 16 (decode GEMV, batched decode, SwiGLU front half).
//
// HBM-bound: every packed weight byte is read exactly once.  The arithmetic runs on the
// matrix cores even at M = 1, because the fp32 VALU cannot keep up with HBM: at 8 TB/s the
// chip has ~2.5 VALU lane-ops per weight and a convert + FMA path needs ~2.4.  Building MFMA
// operands costs 1 op per weight and the MACs are free.
//
// Work decomposition
//   tile   = 128 * LW output columns = 16 lanes x LW packed words (8 * LW columns) per lane
//   K-step = 32 rows = one v_mfma_f32_16x16x32_bf16; lane (lg, ln) = (lane / 16, lane % 16)
//            loads rows 8*lg .. 8*lg+7 of chunk ln, i.e. exactly the K-slice the MFMA B
//            operand wants from that lane
//   unit   = KSTEPS consecutive K-steps inside one quantisation group, all of its loads issued
//            before any of it is consumed
//   wave   = `units` units; workgroup = WAVES waves on one (tile, K-slice, matrix); the grid is
//            (tiles, K-slices, matrices) with all workgroups of a tile on the same XCD
//
// Operand construction.  For rows (k, k+1) and byte p of a packed word, v_perm_b32 builds
// [0, byte_p(row k+1), 0, byte_p(row k)]; `& 0x000F000F | 0x43004300` turns the low nibbles
// into the bf16 pair (128 + q_k, 128 + q_k+1) exactly (0x4300 | q == 128 + q), the same on
// the word shifted by 4 gives the high nibbles.  Each 16x16 MFMA tile is one nibble position
// of one word: its 16 columns are the 16 lanes' chunks.  Zero point and scale are applied
// once per group in fp32:   y += s * (sum (128 + q) x  -  (128 + z) * sum x),
// where sum x comes from one extra MFMA against a B operand of ones.
//
// The M rows of x sit in MFMA rows 4*i + lg' (row m -> lane group m % 4, register m / 4) so
// that for M <= 4 only accumulator register 0 is live in the group flush.
//
// Cross-wave combine goes through LDS.  Cross-workgroup combine: every workgroup of a tile
// except the last one in dispatch order (last K-slice of the last matrix) stores its fp32
// partial to the workspace and exits; the last one (the reducer) polls for those partials,
// two polling rounds in flight at a time, adds them in fixed order
// (deterministic), applies the epilogue and writes y.  A partial slot holds the sentinel
// 0xFFFFFFFF ("empty") until its producer overwrites it, and the reducer puts the sentinel
// back after reading, so the workspace is clean again when the kernel ends.  All slot
// traffic uses agent-scope atomic loads/stores (served at the device coherence point, never
// stale in an XCD's L2) and needs no fences: validity travels with each 32-bit value.  The
// reducer is dispatched after its producers (workgroups are dispatched in linear id order, x fastest), so
// the producers never wait on anything and the poll terminates; it is bounded all the same
// and reports a timeout through the workspace header instead of hanging.
#include "common.h"
#include "kernels.h"
#include "slots.h"

namespace w4a16 {

StreamTune g_stream_tune;

struct StreamParams {
    const uint16_t *x;
    const uint32_t *qw[2];
    const uint32_t *qz[2];
    const uint16_t *sc[2];
    uint16_t *y;
    uint32_t *header;   // workspace header: word 0 = poll timeouts seen
    float *partial;     // [nmat * ksplit][ntiles][2 planes][M * tile columns / 2]: a quad's words 0, 1 and words 2, 3
    int M, K, N;
    int nb;        // N / 8 packed words per row
    int ntiles;    // ceil(N / tile columns)
    int ksplit;    // workgroups along K per tile
    int units;     // units per wave (of the largest slice)
    int slice_units, slice_extra;   // units per K-slice: slice_units, +1 for the first slice_extra slices
    int nmat;      // 1, or 2 for gate/up with the SwiGLU epilogue
    const uint16_t *residual;   // [M, N] bf16 added in the epilogue, or null
    int round_before_add;       // 1: y = bf16(bf16(acc) + R); 0: y = bf16(acc + R)
    const uint16_t *norm_w;     // [K] bf16 RMSNorm weight (RMS kernels only)
    float eps;
    const float *sumsq_in;      // RMS, M == 1: partial sums of x^2 written by the kernel that produced x, or null
    int sumsq_n;
    float *sumsq_out;           // M == 1: sum of squares of this launch's bf16 outputs, one float per column tile, or null
    const float *attn_ml, *attn_acc;   // ATT kernels: the decode attention's partials (StreamExtras)
    int attn_nsplit, attn_hd;
    int spin_limit;
    int skip_publish;   // fault injection for tests: producers keep their partials to themselves
};

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// a0 += sum of squares of the low bf16 halves of v, a1 += of the high halves
__device__ __forceinline__ void sumsq8(const u32x4 v, float &a0, float &a1) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = __builtin_bit_cast(float, v[j] << 16);
        const float hi = __builtin_bit_cast(float, v[j] & 0xFFFF0000u);
        a0 = fmaf(lo, lo, a0);
        a1 = fmaf(hi, hi, a1);
    }
}

template <int LW>
struct Words;
template <>
struct Words<4> { typedef u32x4 type; };
template <>
struct Words<2> { typedef u32x2 type; };
template <>
struct Words<1> { typedef uint32_t type __attribute__((ext_vector_type(1))); };

// LW     packed words per lane per row: the tile is 16 lanes x 8*LW columns = 128*LW columns
// KSTEPS K-steps per unit, WAVES waves per workgroup, MI live accumulator registers (M <= 4*MI)
// RMS    x is RMS-normalised on the fly: every wave computes 1/sqrt(mean(x^2) + eps) of its
//        rows itself (x is K bf16 values, L2-resident) while its weight loads are in
//        flight, and feeds bf16((x * rstd) * norm_w) to the matrix cores.  M <= 4.
// ATT    M == 1: x is the merge of the decode attention's chunk partials, computed by every wave for the 64 rows of
//        its unit (KSTEPS == 2, inside one head) with the merge kernel's arithmetic in the merge kernel's order,
//        so the result is the same bit for bit; the partials are requested ahead of the weights.
template <int LW, int WB, int KSTEPS, int WAVES, int MI, int NMAT, bool RMS, bool ATT = false>
__global__ void __launch_bounds__(WAVES * 64, 2) stream_kernel(const StreamParams p) {
    constexpr int SLOTS = WAVES;   // one LDS slot per wave: a single write round, no read-modify-write
    typedef typename Words<LW>::type wvec;
    constexpr int TC = 128 * LW;            // tile columns
    constexpr int LC = 8 * LW;              // columns per lane
    constexpr int ROWF = LC * 16;           // LDS floats per output row: [ln (16)][LC], 16-byte chunks XOR-swizzled
    constexpr int NCH = LC / 4;             // 16-byte chunks per lane
    constexpr int QPR = TC / 4;             // 4-column quads per output row
    extern __shared__ __attribute__((aligned(16))) float red[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // scalar: addresses built from it stay on the SALU
    const int lg = lane >> 4;
    const int ln = lane & 15;

    // grid = (tiles rounded up to 8, K-slices, matrices).  Workgroups are numbered x fastest and
    // consecutive numbers go to consecutive XCDs, so with gridDim.x a multiple of 8 all workgroups
    // of a tile share an XCD (tile % 8); they are dispatched in that order too, so the reducer,
    // the last K-slice of the last matrix, starts after all of its producers.
    const int kslice = blockIdx.y;
    const int mat = blockIdx.z;
    // Every kernel argument the main path reads is requested here, before the first branch: left to the
    // compiler the scalar loads are issued one use at a time behind the early exits, four dependent
    // round trips to the constant cache before the first weight load is requested.
    {
        const int i0 = p.ntiles, i1 = p.M, i2 = p.K, i3 = p.N, i4 = p.nb, i5 = p.ksplit, i6 = p.units, i7 = p.slice_units,
                  i8 = p.slice_extra, i9 = p.nmat;
        const void *q0 = p.x, *q1 = p.qw[mat], *q2 = p.qz[mat], *q3 = p.sc[mat];
        asm volatile("" ::"s"(i0), "s"(i1), "s"(i2), "s"(i3), "s"(i4), "s"(i5), "s"(i6), "s"(i7), "s"(i8), "s"(i9), "s"(q0),
                     "s"(q1), "s"(q2), "s"(q3));
    }
    const int per_tile = p.nmat * p.ksplit;
    const int tile = blockIdx.x;
    if (tile >= p.ntiles) return;
    const int sub = mat * p.ksplit + kslice;

    const int nchunks = p.nb / LW;
    const int chunk = tile * 16 + ln;
    const int chunk_c = chunk < nchunks ? chunk : nchunks - 1;   // ragged tile: load in range, never written
    // Every load address is a scalar part (matrix base + K-step row offset, SALU) plus one 32-bit
    // per-lane byte offset, so that issuing a unit's 39 loads costs no vector address arithmetic.
    const char *qw_s = reinterpret_cast<const char *>(p.qw[mat]);
    const char *qz_s = reinterpret_cast<const char *>(p.qz[mat]);
    const char *sc_s = reinterpret_cast<const char *>(p.sc[mat]);
    const uint32_t qw_lane = (uint32_t)(((size_t)chunk_c * LW + (size_t)(8 * lg) * p.nb) * sizeof(uint32_t));
    const uint32_t qz_lane = (uint32_t)((size_t)chunk_c * LW * sizeof(uint32_t));
    const uint32_t sc_lane = (uint32_t)((size_t)chunk_c * LC * sizeof(uint16_t));
    const size_t row_bytes = (size_t)p.nb * sizeof(uint32_t);

    // x row held by this lane in the MFMA A operand (A row = ln): m = ln / 4 + 4 * (ln % 4).
    const int am = (ln >> 2) + 4 * (ln & 3);
    const bool a_valid = ((ln & 3) < MI) && (am < p.M);
    const char *x_s = reinterpret_cast<const char *>(p.x);
    const uint32_t x_lane = (uint32_t)(((size_t)(a_valid ? am : 0) * p.K + 8 * lg) * sizeof(uint16_t));

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
    // Kept opaque so the compiler holds them in registers and fuses (v & mask) | magic into
    // one v_and_or_b32 instead of two literal-operand instructions.
    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));

    floatx4 yacc[LC];
#pragma unroll
    for (int t = 0; t < LC; ++t) yacc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // RMSNorm prologue: rstd = 1 / sqrt(mean(x^2) + eps) of the lane's row of x, computed by every
    // wave for itself.  When the kernel that produced x left its sum of squares behind (M == 1,
    // at most 64 pieces) that is one 4-byte load per lane, requested ahead of the weights (loads
    // of one wave return in order) and reduced while they are in flight; otherwise the wave walks
    // x (K bf16 values per row, L2-resident) before it requests its weights.
    float rstd = 0.f;
    float piece = 0.f;
    if constexpr (RMS) {
        if (p.M == 1 && p.sumsq_in) {
            piece = lane < p.sumsq_n ? p.sumsq_in[lane] : 0.f;
        } else {
            float mine = 0.f;
            for (int r = 0; r < p.M; ++r) {   // every lane walks row r, the lanes that feed row r keep its sum
                const u32x4 *row = reinterpret_cast<const u32x4 *>(p.x + (size_t)r * p.K);
                float a0 = 0.f, a1 = 0.f;
                for (int c0 = lane; c0 < (p.K >> 3); c0 += 256) {
                    u32x4 v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        v[i] = c0 + 64 * i < (p.K >> 3) ? row[c0 + 64 * i] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                    for (int i = 0; i < 4; ++i) sumsq8(v[i], a0, a1);
                }
                float a = a0 + a1;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) a += __shfl_xor(a, off);
                if (am == r) mine = a;
            }
            rstd = 1.0f / sqrtf(mine / (float)p.K + p.eps);
        }
    }

    // K-slice `kslice` owns units [ulo, uhi) of the K / (32 * KSTEPS) units: slice_units each, the
    // first slice_extra slices one more; its waves take them round-robin.
    const int ulo = kslice * p.slice_units + (kslice < p.slice_extra ? kslice : p.slice_extra);
    const int uhi = ulo + p.slice_units + (kslice < p.slice_extra ? 1 : 0);
    for (int u = 0; u < p.units; ++u) {
        const int unit = ulo + u * WAVES + wave;
        if (unit >= uhi) break;   // wave-uniform
        const int kstep0 = unit * KSTEPS;
        const int g = kstep0 >> 2;

        wvec w[KSTEPS][8];
        u32x4 av[KSTEPS];
        u32x4 nw[RMS ? KSTEPS : 1];   // norm weights: requested before the packed weights, like x
        if constexpr (RMS) {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s)
                nw[s] = *reinterpret_cast<const u32x4 *>(p.norm_w + (size_t)(kstep0 + s) * 32 + 8 * lg);
        }
        // x first (a wave's loads return in order and the x sum needs every K-step's x), then the weights
        // K-step by K-step, so that K-step s can be consumed while the later ones are still in flight.
        float attn_a[ATT ? kMaxAttnSplit : 1];
        float attn_m = kAttnNegBig, attn_l = 0.f;
        if constexpr (ATT) {
            static_assert(!ATT || (KSTEPS == 2 && MI == 1 && NMAT == 1 && !RMS), "attention merge prologue: plain M = 1 units of 64 rows");
            const int head = (kstep0 * 32) / p.attn_hd;                 // scalar: the unit lies inside one head
            const int e = kstep0 * 32 - head * p.attn_hd + lane;        // this lane's element of the head
            const float *src = p.attn_acc + (size_t)head * p.attn_nsplit * p.attn_hd + e;
#pragma unroll
            for (int c = 0; c < kMaxAttnSplit; ++c) attn_a[c] = c < p.attn_nsplit ? src[(size_t)c * p.attn_hd] : 0.f;
            if (lane < p.attn_nsplit) {                                 // lane c owns chunk c
                const float *ml = p.attn_ml + 2 * ((size_t)head * p.attn_nsplit + lane);
                attn_m = ml[0];
                attn_l = ml[1];
            }
        } else {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s)
                av[s] = *reinterpret_cast<const u32x4 *>(x_s + (size_t)(kstep0 + s) * 32 * sizeof(uint16_t) + x_lane);
        }
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const size_t krow = (size_t)(kstep0 + s) * 32;          // scalar
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w[s][i] = __builtin_nontemporal_load(reinterpret_cast<const wvec *>(qw_s + (krow + i) * row_bytes + qw_lane));
            if constexpr (NMAT == 1 || RMS) __builtin_amdgcn_sched_barrier(0);   // the load clustering would mix the K-steps
        }
        wvec zw;
        u32x4 sv[LW];
        {
            zw = *reinterpret_cast<const wvec *>(qz_s + (size_t)g * row_bytes + qz_lane);
#pragma unroll
            for (int c = 0; c < LW; ++c)
                sv[c] = *reinterpret_cast<const u32x4 *>(sc_s + ((size_t)g * p.N + 8 * c) * sizeof(uint16_t) + sc_lane);
        }
        // Keep every load of the unit above this point: left alone, the scheduler sinks half of
        // them below the first MFMAs to save registers, and a wave then waits for memory twice
        // (GEMV 10.55 -> 10.25 us).  It costs ~27 registers, i.e. the third wave per SIMD, which the
        // plain two-matrix kernel needs more (its grid runs in two rounds), so that one is left alone.
        if constexpr (NMAT == 1 || RMS) __builtin_amdgcn_sched_barrier(0);

        if constexpr (RMS) {
            if (u == 0 && p.M == 1 && p.sumsq_in) {
                float a = piece;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) a += __shfl_xor(a, off);
                rstd = 1.0f / sqrtf(a / (float)p.K + p.eps);
            }
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float x_lo = __builtin_bit_cast(float, av[s][j] << 16);
                    const float x_hi = __builtin_bit_cast(float, av[s][j] & 0xFFFF0000u);
                    const float w_lo = __builtin_bit_cast(float, nw[s][j] << 16);
                    const float w_hi = __builtin_bit_cast(float, nw[s][j] & 0xFFFF0000u);
                    av[s][j] = pack_bf16x2((x_lo * rstd) * w_lo, (x_hi * rstd) * w_hi);
                }
            }
        }
        if constexpr (ATT) {
            // out[e] = sum_c acc_c[e] 2^(m_c - M) / sum_c l_c 2^(m_c - M), as in attn_combine_kernel
            const float mn = wave_reduce<true>(attn_m);
            const float wgt = lane < p.attn_nsplit ? exp2f(attn_m - mn) : 0.f;
            const float inv_l = 1.0f / wave_reduce<false>(attn_l * wgt);
            float as = 0.f;
#pragma unroll
            for (int c = 0; c < kMaxAttnSplit; ++c)
                as = fmaf(attn_a[c], __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wgt), c)), as);
            // lane i holds row i of the unit; the MFMA operand wants 8 consecutive rows in lanes 0, 16, 32, 48: through
            // the wave's own part of the combine buffer (LDS operations of one wave are carried out in order)
            uint16_t *stage = reinterpret_cast<uint16_t *>(red + wave * (p.M * ROWF));
            stage[lane] = float_to_bf16_bits(as * inv_l);
            asm volatile("" ::: "memory");
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) av[s] = *reinterpret_cast<const u32x4 *>(stage + 32 * s + 8 * lg);
            asm volatile("" ::: "memory");
        }
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            if (!a_valid) av[s] = u32x4{0u, 0u, 0u, 0u};
        {
            floatx4 xs = floatx4{0.f, 0.f, 0.f, 0.f};
    #pragma unroll
            for (int s = 0; s < KSTEPS; ++s)
                xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[s]), ones, xs, 0, 0, 0);

            // WB packed words (8 * WB MFMA tiles) at a time: K-steps outer so that work starts as
            // soon as a K-step's loads have landed, then the group flush of those words.
            // acc[cc * 8 + pos]: word cb + cc, nibble position pos (= 2 * byte + nibble-in-byte).
    #pragma unroll
            for (int cb = 0; cb < LW; cb += WB) {
                floatx4 acc[8 * WB];
    #pragma unroll
                for (int t = 0; t < 8 * WB; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
    #pragma unroll
                for (int s = 0; s < KSTEPS; ++s) {
                    const bf16x8 a = __builtin_bit_cast(bf16x8, av[s]);
    #pragma unroll
                    for (int cc = 0; cc < WB; ++cc) {
                        const int c = cb + cc;
    #pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            const uint32_t sel = 0x0C000C00u | ((4u + b) << 16) | (uint32_t)b;
                            u32x4 lo, hi;
    #pragma unroll
                            for (int v = 0; v < 4; ++v) {
                                const uint32_t pr = __builtin_amdgcn_perm(w[s][2 * v + 1][c], w[s][2 * v][c], sel);
                                lo[v] = (pr & nib_mask) | magic;
                                hi[v] = ((pr >> 4) & nib_mask) | magic;
                            }
                            const int t = cc * 8 + 2 * b;
                            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, lo), acc[t], 0, 0, 0);
                            acc[t + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, hi), acc[t + 1], 0, 0, 0);
                        }
                    }
                    // Nothing of K-step s + 1 moves above this point: left alone, the scheduler interleaves the
                    // operand construction of later K-steps with the first MFMAs and the wave then waits for
                    // three quarters of its loads before it starts.
                    if constexpr (NMAT == 1 || RMS) __builtin_amdgcn_sched_barrier(0);
                }
                // Group flush.  Nibble positions (q, q + 4) of a word are natural columns (2q, 2q + 1),
                // i.e. the two halves of scale word q; (zw >> 4q) & 0x000F000F | 0x43004300 is the bf16
                // pair (128 + z) of the same two columns.  yacc[c * 8 + j] is natural column 8c + j.
    #pragma unroll
                for (int cc = 0; cc < WB; ++cc) {
                    const int c = cb + cc;
    #pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t zp = ((zw[c] >> (4 * q)) & nib_mask) | magic;
                        const uint32_t sw = sv[c][q];
                        const float z_lo = __builtin_bit_cast(float, zp << 16), z_hi = __builtin_bit_cast(float, zp & 0xFFFF0000u);
                        const float s_lo = __builtin_bit_cast(float, sw << 16), s_hi = __builtin_bit_cast(float, sw & 0xFFFF0000u);
    #pragma unroll
                        for (int i = 0; i < MI; ++i) {
                            yacc[c * 8 + 2 * q][i] = fmaf(s_lo, fmaf(-z_lo, xs[i], acc[cc * 8 + q][i]), yacc[c * 8 + 2 * q][i]);
                            yacc[c * 8 + 2 * q + 1][i] = fmaf(s_hi, fmaf(-z_hi, xs[i], acc[cc * 8 + q + 4][i]), yacc[c * 8 + 2 * q + 1][i]);
                        }
                    }
                }
            }
        }
    }

    const int nprod = per_tile - 1;
    const bool reducer = (sub == nprod);
    const int nquads = p.M * QPR;
    const int col0 = tile * TC;
    const size_t slice_stride = (size_t)p.ntiles * nquads * 4;                 // floats per (mat, kslice)
    float *tile_partial = p.partial + (size_t)tile * nquads * 4;
    const size_t plane = (size_t)nquads * 2;   // a tile's slots are two planes of 8 bytes per quad

    // The reducer's first polling round is issued before the LDS combine, so that its latency
    // (one trip to L2 per slot) is hidden behind the combine and its barriers.
    u32x4 va[8], vb[8];   // the two polling rounds a reducer thread keeps in flight
    const bool prefetched = reducer && nprod > 0 && (int)threadIdx.x < nquads;
    if (prefetched) {
        // every round issues all eight loads (a slot index past the last producer is clamped to it and the copy
        // ignored): no load of a round is predicated, so no register of a round can hold a stale value
#pragma unroll
        for (int j = 0; j < 8; ++j)
            va[j] = slot_load_planes(tile_partial + (size_t)threadIdx.x * 2 + (j < nprod ? j : nprod - 1) * slice_stride, plane);
    }

    // ---- cross-wave combine in LDS: red[slot][m][ln][LC], moved as 16-byte chunks (4 columns).  Chunk jj
    // of lane ln sits at position jj ^ key(ln), key = (ln * LC / 32) % NCH, so that 8 neighbouring
    // lanes cover all 32 banks both when a lane writes its chunks and when 8 threads read 8 neighbouring quads.
    const int slot_stride = p.M * ROWF;
    {
        float *dst = red + wave * slot_stride + ln * LC;
        const int key = (ln * LC / 32) % NCH;
#pragma unroll
        for (int jj = 0; jj < NCH; ++jj) {
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int m = lg + 4 * i;
                if (m < p.M)
                    *reinterpret_cast<floatx4 *>(dst + m * ROWF + 4 * (jj ^ key)) =
                        floatx4{yacc[4 * jj][i], yacc[4 * jj + 1][i], yacc[4 * jj + 2][i], yacc[4 * jj + 3][i]};
            }
        }
    }
    __syncthreads();

    // ---- workgroup result in 4-column quads; producers publish, the reducer gathers ----
    for (int e = threadIdx.x; e < nquads; e += WAVES * 64) {
        const int m = e / QPR;
        const int col = (e % QPR) * 4;
        floatx4 own = floatx4{0.f, 0.f, 0.f, 0.f};
        {
            const int qi = e % QPR, qln = qi / NCH, qjj = qi % NCH;
            const float *src = red + m * ROWF + qln * LC + 4 * (qjj ^ ((qln * LC / 32) % NCH));
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) own += *reinterpret_cast<const floatx4 *>(src + s * slot_stride);
        }
        float *slot0 = tile_partial + (size_t)e * 2;   // words 0, 1 here, words 2, 3 one plane further
        if (!reducer) {
            u32x4 bits = __builtin_bit_cast(u32x4, own);
#pragma unroll
            for (int q = 0; q < 4; ++q) bits[q] = bits[q] == kEmpty ? 0x7FC00000u : bits[q];   // keep the sentinel unique
            if (!p.skip_publish) slot_store_planes(slot0 + sub * slice_stride, plane, bits);
            continue;
        }
        // Reducer: fetch the producers' slots eight at a time (all loads of a round in flight
        // together) until they are all filled, then hand the slots back.  Two rounds are kept in
        // flight, half a round trip apart, so that a partial is noticed about one round trip after
        // it was published instead of up to two.
        floatx4 sum0 = floatx4{0.f, 0.f, 0.f, 0.f}, sum1 = floatx4{0.f, 0.f, 0.f, 0.f};
        for (int s0 = 0; s0 < nprod; s0 += 8) {
#define W4A16_POLL_ISSUE(dst)                                                                 \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) dst[j] = slot_load_planes(slot0 + (s0 + j < nprod ? s0 + j : nprod - 1) * slice_stride, plane)
#define W4A16_POLL_FULL(src, ok)                                                              \
    ok = true;                                                                                \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) if (s0 + j < nprod) ok = ok && slot_full(src[j])
#define W4A16_POLL_TAKE(src)                                                                  \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) if (s0 + j < nprod) {                       \
        if (NMAT == 2 && s0 + j >= p.ksplit) sum1 += __builtin_bit_cast(floatx4, src[j]);     \
        else sum0 += __builtin_bit_cast(floatx4, src[j]);                                     \
    }
            if (!(prefetched && s0 == 0 && e == (int)threadIdx.x)) {   // else: va holds the early first round
                W4A16_POLL_ISSUE(va);
            }
            int spins = 0;
            bool ok;
            for (;;) {
                W4A16_POLL_ISSUE(vb);
                W4A16_POLL_FULL(va, ok);
                if (ok || ++spins > p.spin_limit) {
                    W4A16_POLL_TAKE(va);
                    break;
                }
                __builtin_amdgcn_s_sleep(POLL_SLEEP);
                W4A16_POLL_ISSUE(va);
                W4A16_POLL_FULL(vb, ok);
                if (ok) {
                    W4A16_POLL_TAKE(vb);
                    break;
                }
                __builtin_amdgcn_s_sleep(POLL_SLEEP);
            }
            if (!ok) __hip_atomic_store(p.header, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#undef W4A16_POLL_ISSUE
#undef W4A16_POLL_FULL
#undef W4A16_POLL_TAKE
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (s0 + j < nprod) slot_store_planes(slot0 + (s0 + j) * slice_stride, plane, u32x4{kEmpty, kEmpty, kEmpty, kEmpty});
        }
        floatx4 out;
        if (NMAT == 2) {
            sum1 += own;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float gate = bf16_bits_to_float(float_to_bf16_bits(sum0[q]));
                const float up = bf16_bits_to_float(float_to_bf16_bits(sum1[q]));
                out[q] = silu_tanh(gate) * up;
            }
        } else {
            out = sum0 + own;
        }
        if (p.residual && col0 + col < p.N) {
            const uint2 r = *reinterpret_cast<const uint2 *>(p.residual + (size_t)m * p.N + col0 + col);
            if (p.round_before_add) {
#pragma unroll
                for (int q = 0; q < 4; ++q) out[q] = bf16_bits_to_float(float_to_bf16_bits(out[q]));
            }
            out[0] += __builtin_bit_cast(float, r.x << 16);
            out[1] += __builtin_bit_cast(float, r.x & 0xFFFF0000u);
            out[2] += __builtin_bit_cast(float, r.y << 16);
            out[3] += __builtin_bit_cast(float, r.y & 0xFFFF0000u);
        }
        uint2 o;
        o.x = pack_bf16x2(out[0], out[1]);
        o.y = pack_bf16x2(out[2], out[3]);
        const bool in_range = col0 + col < p.N;
        if (in_range) *reinterpret_cast<uint2 *>(p.y + (size_t)m * p.N + col0 + col) = o;
        if (p.sumsq_out && p.M == 1) {
            // M == 1: the tile's quads are exactly the lanes of wave 0 (one trip through this loop)
            float sq = 0.f;
            if (in_range) {
                const float r0 = __builtin_bit_cast(float, o.x << 16), r1 = __builtin_bit_cast(float, o.x & 0xFFFF0000u);
                const float r2 = __builtin_bit_cast(float, o.y << 16), r3 = __builtin_bit_cast(float, o.y & 0xFFFF0000u);
                sq = fmaf(r0, r0, fmaf(r1, r1, fmaf(r2, r2, r3 * r3)));
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
            if (threadIdx.x == 0) p.sumsq_out[tile] = sq;
        }
    }
}

// Launch shape.  Measured on MI355X (K = 4096, N = 11008): 256-column tiles (8-byte loads),
// 8 waves per workgroup and one unit per wave are the fastest, which makes the K-split
// K / 1024.  All workgroups must be resident at once (one 8-wave workgroup per CU at these
// register counts): a grid beyond 256 workgroups runs in two rounds and takes 17 us instead of
// 10.7 us, and a deeper split within 256 (5 instead of 4) is slower too, because every extra
// producer adds partial traffic to the reducer's critical path.  A long K with few tiles (the FFN down projection, K = 14336, N = 4096: 16 tiles)
// needs the deep split to put a workgroup on most CUs: split 14 (224 workgroups) beats split 7
// by 9 %, so the split is only capped at 16 (two polling rounds of the reducer) for M <= 4.
// For M > 4 the fp32 partials are M times larger and the cap is 4 (M = 16: split 4 16.3 us,
// split 8 32.6 us, split 2 19.4 us), more units per wave instead.
StreamPlan plan_stream(int M, int K, int N, bool fixed_shape) {
    StreamPlan pl;
    pl.mi = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
    const int nksteps = K / 32;
    pl.lw = 2;
    pl.ksteps = 4;
    pl.waves = 8;
    pl.units = 1;
    if (g_stream_tune.lw && !fixed_shape) pl.lw = g_stream_tune.lw == 1 ? 1 : 2;
    if (g_stream_tune.ksteps) pl.ksteps = g_stream_tune.ksteps == 2 ? 2 : 4;
    if (g_stream_tune.waves && !fixed_shape) pl.waves = g_stream_tune.waves == 4 ? 4 : 8;
    pl.ntiles = (N + 128 * pl.lw - 1) / (128 * pl.lw);
    // Few tiles and a short K (e.g. a 4096 x 4096 projection: 16 tiles, 64 workgroups): halve the
    // unit so that twice as many workgroups share the stream (9.1 us instead of 10.1 us there).
    if (!g_stream_tune.ksteps && M <= 4 && pl.ntiles * ((nksteps / 4 + pl.waves - 1) / pl.waves) < 128) pl.ksteps = 2;
    const int nunits = nksteps / pl.ksteps;   // K % 128 == 0, so this is exact for 2 and 4 K-steps per unit
    if (g_stream_tune.ksplit) {
        pl.ksplit = g_stream_tune.ksplit;
    } else if (g_stream_tune.units) {
        pl.ksplit = (nunits + pl.waves * g_stream_tune.units - 1) / (pl.waves * g_stream_tune.units);
    } else {
        // one unit per wave while the split stays under its cap
        const int max_split = M <= 4 ? 16 : 4;
        pl.ksplit = (nunits + pl.waves - 1) / pl.waves;
        if (pl.ksplit > max_split) pl.ksplit = max_split;
    }
    if (pl.ksplit > kMaxKSplit) pl.ksplit = kMaxKSplit;
    if (pl.ksplit > nunits) pl.ksplit = nunits;
    if (pl.ksplit < 1) pl.ksplit = 1;
    const int per_slice = (nunits + pl.ksplit - 1) / pl.ksplit;   // largest slice
    pl.units = (per_slice + pl.waves - 1) / pl.waves;
    return pl;
}

bool stream_attn_fusable(int K, int N, int head_dim, int nsplit) {
    if (head_dim <= 0 || head_dim % 64 != 0 || K % head_dim != 0 || nsplit < 2 || nsplit > kMaxAttnSplit) return false;
    const StreamPlan pl = plan_stream(1, K, N);
    return pl.lw == 2 && pl.ksteps == 2 && pl.waves == 8;   // units of 64 rows: a unit never straddles two heads
}

template <int LW, int WB, int KSTEPS, int WAVES, int MI, int NMAT, bool RMS = false, bool ATT = false>
static hipError_t launch_one(const StreamParams &p, dim3 grid, hipStream_t stream) {
    const size_t lds = (size_t)WAVES * p.M * 8 * LW * 16 * sizeof(float);   // 128 KB at M = 16, LW = 2, 8 waves
    if (lds > 64 * 1024) {   // more than 64 KB of dynamic LDS needs the attribute (per device, so set it every time)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&stream_kernel<LW, WB, KSTEPS, WAVES, MI, NMAT, RMS, ATT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((stream_kernel<LW, WB, KSTEPS, WAVES, MI, NMAT, RMS, ATT>), grid, dim3(WAVES * 64), lds, stream, p);
    return hipGetLastError();
}

template <int LW, int WB, int KSTEPS, int WAVES>
static hipError_t launch_mi(int mi, const StreamParams &p, dim3 grid, hipStream_t stream) {
    if (p.norm_w)   // M <= 4 checked by the caller
        return p.nmat == 2 ? launch_one<LW, WB, KSTEPS, WAVES, 1, 2, true>(p, grid, stream)
                           : launch_one<LW, WB, KSTEPS, WAVES, 1, 1, true>(p, grid, stream);
    if (p.nmat == 2) return launch_one<LW, WB, KSTEPS, WAVES, 1, 2>(p, grid, stream);
    switch (mi) {
        case 1: return launch_one<LW, WB, KSTEPS, WAVES, 1, 1>(p, grid, stream);
        case 2: return launch_one<LW, WB, KSTEPS, WAVES, 2, 1>(p, grid, stream);
        default: return launch_one<LW, WB, KSTEPS, WAVES, 4, 1>(p, grid, stream);
    }
}

template <int LW, int WB, int KSTEPS>
static hipError_t launch_waves(int waves, int mi, const StreamParams &p, dim3 grid, hipStream_t stream) {
    return waves == 4 ? launch_mi<LW, WB, KSTEPS, 4>(mi, p, grid, stream) : launch_mi<LW, WB, KSTEPS, 8>(mi, p, grid, stream);
}

template <int LW, int WB>
static hipError_t launch_ksteps(int ksteps, int waves, int mi, const StreamParams &p, dim3 grid, hipStream_t stream) {
    return ksteps == 2 ? launch_waves<LW, WB, 2>(waves, mi, p, grid, stream) : launch_waves<LW, WB, 4>(waves, mi, p, grid, stream);
}

hipError_t launch_stream(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                         const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                         uint16_t *y, int M, int K, int N, void *workspace, hipStream_t stream,
                         const StreamExtras &extras) {
    // the chained sums of squares count one float per 256-column tile: those launches keep that shape whatever the tune keys say
    const StreamPlan pl = plan_stream(M, K, N, extras.sumsq_out != nullptr || extras.sumsq_in != nullptr);
    StreamParams p;
    p.x = x;
    p.qw[0] = reinterpret_cast<const uint32_t *>(qweight);
    p.qz[0] = reinterpret_cast<const uint32_t *>(qzeros);
    p.sc[0] = scales;
    p.nmat = up_qweight ? 2 : 1;
    p.qw[1] = reinterpret_cast<const uint32_t *>(up_qweight ? up_qweight : qweight);
    p.qz[1] = reinterpret_cast<const uint32_t *>(up_qzeros ? up_qzeros : qzeros);
    p.sc[1] = up_scales ? up_scales : scales;
    p.y = y;
    p.header = reinterpret_cast<uint32_t *>(workspace);
    p.partial = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + kHeaderBytes);
    p.M = M;
    p.K = K;
    p.N = N;
    p.nb = N / 8;
    p.ntiles = pl.ntiles;
    p.ksplit = pl.ksplit;
    p.units = pl.units;
    p.slice_units = (K / 32 / pl.ksteps) / pl.ksplit;
    p.slice_extra = (K / 32 / pl.ksteps) % pl.ksplit;
    p.residual = extras.residual;
    p.round_before_add = extras.round_before_add;
    p.norm_w = extras.norm_w;
    p.eps = extras.eps;
    p.sumsq_in = extras.sumsq_in;
    p.sumsq_n = extras.sumsq_n;
    p.sumsq_out = extras.sumsq_out;
    p.attn_ml = extras.attn_ml;
    p.attn_acc = extras.attn_acc;
    p.attn_nsplit = extras.attn_nsplit;
    p.attn_hd = extras.attn_hd;
    p.skip_publish = g_stream_tune.skip_publish;
    p.spin_limit = g_stream_tune.spin_limit > 0 ? g_stream_tune.spin_limit : (1 << 18);
    const dim3 grid(((pl.ntiles + 7) / 8) * 8, pl.ksplit, p.nmat);
    if (extras.attn_acc) {   // x comes from the attention partials: one instantiation, shapes checked by stream_attn_fusable
        if (M != 1 || up_qweight || extras.norm_w || !extras.attn_ml ||
            !stream_attn_fusable(K, N, extras.attn_hd, extras.attn_nsplit))
            return hipErrorInvalidValue;
        return launch_one<2, 2, 2, 8, 1, 1, false, true>(p, grid, stream);
    }
    return pl.lw == 1 ? launch_ksteps<1, 1>(pl.ksteps, pl.waves, pl.mi, p, grid, stream)
                      : launch_ksteps<2, 2>(pl.ksteps, pl.waves, pl.mi, p, grid, stream);
}

// Workspace reset: header words zero, every partial slot "empty".
__global__ void fill_workspace_kernel(uint32_t *p, size_t nwords, size_t header_words) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nwords; i += (size_t)gridDim.x * blockDim.x)
        p[i] = i < header_words ? 0u : kEmpty;
}

hipError_t launch_fill_workspace(void *ptr, size_t bytes, hipStream_t stream) {
    const size_t nwords = bytes / 4;
    int grid = (int)((nwords + 255) / 256);
    if (grid > 4096) grid = 4096;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(fill_workspace_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<uint32_t *>(ptr), nwords,
                       kHeaderBytes / 4);
    return hipGetLastError();
}

}  // namespace w4a16
