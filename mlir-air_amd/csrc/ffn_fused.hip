// Decode SwiGLU FFN (batch 1) as one persistent kernel: gate/up GEMV + SwiGLU, then the down GEMV.
//
// Two back-to-back streaming launches leave HBM idle twice: while the first kernel's split-K
// reduction drains and while the second kernel's first loads are in flight.  Here every wave runs
// a three-unit pipeline - its gate unit, its up unit, its down unit (a unit = 128 rows x 256 columns
// of one matrix, as in the streaming kernel) - and requests the weights of the down unit as soon as
// the workgroup's gate/up sums have left LDS.  Those weights do not depend on anything the kernel
// computes, so they stream in while the SwiGLU reduction runs; only the 128 values of h that the
// unit multiplies have to wait for it.
//
// Grid: G workgroups of 8 waves, one per CU, G = tilesA * splitA = tilesB * splitB, where a tile
// is 256 output columns (tilesA = H / 256, tilesB = E / 256) and split* the K-slices per tile.
// Workgroup w is (tile w % tilesA, slice w / tilesA) of the gate/up phase and (tile w % tilesB,
// slice w / tilesB) of the down phase; wave v owns unit slice * units_per_slice + v in both.
//
// Cross-workgroup traffic uses the sentinel slots of slots.h, all inside the caller's workspace
// (every word 0xFFFFFFFF between calls):
//   partialA  [2 * (splitA - 1)][tilesA][2 planes][64 quads / 2]   gate and up partials of the producers
//   partialB  [splitB - 1][tilesB][2 planes][64 quads / 2]
//   hpriv     [tilesB][H / 2] words                  one private copy of h (bf16 pairs) per down tile
// The reducer of a gate/up tile (last slice = highest workgroup ids = dispatched last) adds the
// partials in fixed order, applies SwiGLU and writes its 256 values of h into all tilesB copies;
// each 128-value chunk of a copy has exactly one consumer wave, which polls it, takes it and puts
// the sentinel back - the same single-consumer protocol as the partial slots, so the workspace is
// clean again when the kernel ends.  Waits are bounded (spin_limit) and report through the
// workspace header instead of hanging.
//
// Progress: producers never wait before they publish; gate/up reducers wait only for producers;
// down units wait only for gate/up reducers; down reducers wait only for down producers.  All G
// workgroups must be able to become resident (G <= number of CUs, checked by the host), so two
// instances running at the same time on one GPU can starve each other into the timeout path.
#include "common.h"
#include "kernels.h"
#include "slots.h"

namespace w4a16 {

typedef uint32_t u32x2f __attribute__((ext_vector_type(2)));

struct FfnParams {
    const uint16_t *x;          // [E]
    const uint32_t *qw[3];      // gate, up [E, H/8]; down [H, E/8]
    const uint32_t *qz[3];
    const uint16_t *sc[3];
    const uint16_t *residual;   // [E] added to y, or null
    const uint16_t *norm_w;     // RMS kernels: [E] bf16, x is replaced by bf16((x * rstd) * norm_w)
    const float *sumsq_in;      // RMS kernels: partial sums of x^2 left by the kernel that produced x (<= 64)
    int sumsq_n;
    float eps;
    uint16_t *y;                // [E]
    uint16_t *h_out;            // [H] or null
    float *sumsq_out;           // [E / 256] or null: sum of squares of the bf16 y values of each 256-column tile
    uint32_t *header;
    float *partialA;
    float *partialB;
    uint32_t *hpriv;
    int E, H;
    int tilesA, splitA, upsA;   // upsA = units per slice (<= 8)
    int tilesB, splitB, upsB;
    int spin_limit;
};

struct UnitRegs {
    u32x2f w[4][8];   // 4 K-steps x 8 rows, two packed words (16 columns) per lane
    u32x2f zw;
    u32x4 sv[2];
};

// The loads of one unit: rows [128 * unit, +128) of a [K, N/8] matrix, the lane's two words of tile `tile`.
// Zero points and scales are requested first (a wave's loads return in order, and they are small), the
// weights K-step by K-step with the order pinned, so that compute_unit can start on K-step 0 while the
// later ones are still in flight (left alone, the load clustering mixes the K-steps).
__device__ __forceinline__ void load_unit_meta(UnitRegs &u, const uint32_t *qz, const uint16_t *sc, int N, int tile, int unit,
                                               int ln) {
    const int nb = N >> 3;
    const size_t word = (size_t)(tile * 16 + ln) * 2;
    u.zw = *reinterpret_cast<const u32x2f *>(qz + (size_t)unit * nb + word);
#pragma unroll
    for (int c = 0; c < 2; ++c)
        u.sv[c] = *reinterpret_cast<const u32x4 *>(sc + (size_t)unit * N + (size_t)(tile * 16 + ln) * 16 + 8 * c);
}
__device__ __forceinline__ void load_unit_weights(UnitRegs &u, const uint32_t *qw, int N, int tile, int unit, int lg, int ln) {
    const int nb = N >> 3;
    const size_t word = (size_t)(tile * 16 + ln) * 2;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const size_t row = (size_t)unit * 128 + s * 32 + 8 * lg + i;
            u.w[s][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x2f *>(qw + row * nb + word));
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}
__device__ __forceinline__ void load_unit(UnitRegs &u, const uint32_t *qw, const uint32_t *qz, const uint16_t *sc, int N,
                                          int tile, int unit, int lg, int ln) {
    load_unit_meta(u, qz, sc, N, tile, unit, ln);
    load_unit_weights(u, qw, N, tile, unit, lg, ln);
}

// yacc[j] += row 0 of x . W for the lane's 16 columns (natural order), as in the streaming kernel:
// y += s * (sum (128 + q) x - (128 + z) sum x).
__device__ __forceinline__ void compute_unit(const UnitRegs &u, const u32x4 (&av)[4], float (&yacc)[16], uint32_t nib_mask,
                                             uint32_t magic) {
    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
    floatx4 xs = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[s]), ones, xs, 0, 0, 0);
    floatx4 acc[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, av[s]);
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint32_t sel = 0x0C000C00u | ((4u + b) << 16) | (uint32_t)b;
                u32x4 lo, hi;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint32_t pr = __builtin_amdgcn_perm(u.w[s][2 * v + 1][c], u.w[s][2 * v][c], sel);
                    lo[v] = (pr & nib_mask) | magic;
                    hi[v] = ((pr >> 4) & nib_mask) | magic;
                }
                const int t = c * 8 + 2 * b;
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, lo), acc[t], 0, 0, 0);
                acc[t + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, hi), acc[t + 1], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);   // K-step s + 1 stays below: its operands are built when its loads have landed
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t zp = ((u.zw[c] >> (4 * q)) & nib_mask) | magic;
            const uint32_t sw = u.sv[c][q];
            const float z_lo = __builtin_bit_cast(float, zp << 16), z_hi = __builtin_bit_cast(float, zp & 0xFFFF0000u);
            const float s_lo = __builtin_bit_cast(float, sw << 16), s_hi = __builtin_bit_cast(float, sw & 0xFFFF0000u);
            yacc[c * 8 + 2 * q] = fmaf(s_lo, fmaf(-z_lo, xs[0], acc[c * 8 + q][0]), yacc[c * 8 + 2 * q]);
            yacc[c * 8 + 2 * q + 1] = fmaf(s_hi, fmaf(-z_hi, xs[0], acc[c * 8 + q + 4][0]), yacc[c * 8 + 2 * q + 1]);
        }
    }
}

// One wave's 256-column row into its LDS slot (16-byte chunks, XOR-swizzled as in the streaming kernel).
__device__ __forceinline__ void lds_put(float *slot, const float (&yacc)[16], int lg, int ln) {
    if (lg != 0) return;   // row 0 of the MFMA result lives in lanes 0..15
    const int key = (ln >> 1) & 3;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
        *reinterpret_cast<floatx4 *>(slot + ln * 16 + 4 * (jj ^ key)) =
            floatx4{yacc[4 * jj], yacc[4 * jj + 1], yacc[4 * jj + 2], yacc[4 * jj + 3]};
}

// Sum over the 8 wave slots of quad `qi` (columns 4 qi .. 4 qi + 3).
__device__ __forceinline__ floatx4 lds_sum(const float *base, int qi) {
    const int qln = qi >> 2, qjj = qi & 3;
    const float *src = base + qln * 16 + 4 * (qjj ^ ((qln >> 1) & 3));
    floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 8; ++w) s += *reinterpret_cast<const floatx4 *>(src + w * 256);
    return s;
}

__device__ __forceinline__ u32x4 keep_sentinel_unique(floatx4 v) {
    u32x4 bits = __builtin_bit_cast(u32x4, v);
#pragma unroll
    for (int q = 0; q < 4; ++q) bits[q] = bits[q] == kEmpty ? 0x7FC00000u : bits[q];
    return bits;
}

// Adds the `n` slots base + j * stride (j < split into sum0, the rest into sum1) once they are all
// filled, then empties them.  A tile's 64 slots are two planes of 128 floats (slot_store_planes): base is
// the tile's region + 2 * lane.  Two polling rounds in flight.  Returns false after spin_limit rounds.
// Every round issues the same eight slot loads whatever n is (slots past the end re-read the last
// one and are masked out of the test and the sum), so that the number of loads in flight at each
// wait is fixed; with loads skipped by branches, stale registers were sporadically accepted as
// filled slots (about one call in a thousand).
__device__ __forceinline__ bool gather(float *base, size_t stride, int n, int split, floatx4 &sum0, floatx4 &sum1,
                                       int spin_limit) {
    bool all_ok = true;
    for (int s0 = 0; s0 < n; s0 += 8) {
        u32x4 va[8], vb[8];
        const float *addr[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) addr[j] = base + (size_t)(s0 + j < n ? s0 + j : n - 1) * stride;
#define FFN_ISSUE(dst) _Pragma("unroll") for (int j = 0; j < 8; ++j) dst[j] = slot_load_planes(addr[j], 128)
#define FFN_FULL(src, ok) ok = true; _Pragma("unroll") for (int j = 0; j < 8; ++j) ok = ok && slot_full(src[j])
#define FFN_TAKE(src)                                                                         \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                           \
        const floatx4 v = __builtin_bit_cast(floatx4, src[j]);                                \
        const bool live = s0 + j < n, second = s0 + j >= split;                               \
        _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                       \
            sum0[q] += live && !second ? v[q] : 0.f;                                          \
            sum1[q] += live && second ? v[q] : 0.f;                                           \
        }                                                                                     \
    }
        FFN_ISSUE(va);
        int spins = 0;
        bool ok;
        for (;;) {
            FFN_ISSUE(vb);
            FFN_FULL(va, ok);
            if (ok || ++spins > spin_limit) {
                FFN_TAKE(va);
                break;
            }
            __builtin_amdgcn_s_sleep(POLL_SLEEP);
            FFN_ISSUE(va);
            FFN_FULL(vb, ok);
            if (ok) {
                FFN_TAKE(vb);
                break;
            }
            __builtin_amdgcn_s_sleep(POLL_SLEEP);
        }
#undef FFN_ISSUE
#undef FFN_FULL
#undef FFN_TAKE
        all_ok = all_ok && ok;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (s0 + j < n) slot_store_planes(base + (size_t)(s0 + j) * stride, 128, u32x4{kEmpty, kEmpty, kEmpty, kEmpty});
    }
    return all_ok;
}

// RMS: x is RMS-normalised on the fly, as in the streaming kernel's prologue for M = 1 (the sum of
// squares comes from the launch that produced x; the norm weights are requested ahead of the packed
// weights because one wave's loads return in order).
template <bool RMS>
__global__ void __launch_bounds__(512, 2) ffn_fused_kernel(const FfnParams p) {
    // gate slots [8][256], up slots [8][256], down slots [8][256]
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    const int wg = blockIdx.x;
    const int tileA = wg % p.tilesA, sliceA = wg / p.tilesA;
    const int tileB = wg % p.tilesB, sliceB = wg / p.tilesB;
    const bool hasA = wave < p.upsA, hasB = wave < p.upsB;
    const int unitA = sliceA * p.upsA + wave, unitB = sliceB * p.upsB + wave;
    const bool reducerA = sliceA == p.splitA - 1, reducerB = sliceB == p.splitB - 1;
    const bool gather_wave = reducerA && wave == 0;   // its poll results must not queue behind a weight prefetch

    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));
    const bool a_valid = ln == 0;   // x sits in MFMA row 0

    // ---- gate and up units: everything requested up front ----
    UnitRegs r0, r1;
    u32x4 av[4];
    u32x4 nw[RMS ? 4 : 1];
    float piece = 0.f;
    if (hasA) {
        if constexpr (RMS) {
            piece = lane < p.sumsq_n ? p.sumsq_in[lane] : 0.f;
#pragma unroll
            for (int s = 0; s < 4; ++s)
                nw[s] = *reinterpret_cast<const u32x4 *>(p.norm_w + (size_t)unitA * 128 + s * 32 + 8 * lg);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
            av[s] = *reinterpret_cast<const u32x4 *>(p.x + (size_t)unitA * 128 + s * 32 + 8 * lg);
        load_unit_meta(r0, p.qz[0], p.sc[0], p.H, tileA, unitA, ln);
        load_unit_meta(r1, p.qz[1], p.sc[1], p.H, tileA, unitA, ln);
        __builtin_amdgcn_sched_barrier(0);
        load_unit_weights(r0, p.qw[0], p.H, tileA, unitA, lg, ln);
        load_unit_weights(r1, p.qw[1], p.H, tileA, unitA, lg, ln);
    }
    __builtin_amdgcn_sched_barrier(0);
    float yg[16], yu[16], yd[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) yg[j] = yu[j] = yd[j] = 0.f;
    if (hasA) {
        if constexpr (RMS) {
            float a = piece;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) a += __shfl_xor(a, off);
            const float rstd = 1.0f / sqrtf(a / (float)p.E + p.eps);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
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
#pragma unroll
        for (int s = 0; s < 4; ++s)
            if (!a_valid) av[s] = u32x4{0u, 0u, 0u, 0u};
        compute_unit(r0, av, yg, nib_mask, magic);
    }
    if (hasA) compute_unit(r1, av, yu, nib_mask, magic);

    // ---- gate/up: cross-wave combine ----
    // The sums are read from LDS between two barriers, while no wave of the workgroup has a global
    // load in flight.  (Measured: with the down unit's weights already on their way in the other
    // waves, 128-bit LDS reads of the summing wave sporadically came back incomplete - some lanes of
    // the destination registers kept their previous contents - whenever those registers had the
    // same numbers as the other waves' load destinations.  Requesting the weights only after the
    // second barrier removes the overlap by construction.)
    lds_put(red + wave * 256, yg, lg, ln);
    lds_put(red + 2048 + wave * 256, yu, lg, ln);
    __syncthreads();
    const int nprodA = p.splitA - 1;
    floatx4 own0 = floatx4{0.f, 0.f, 0.f, 0.f}, own1 = floatx4{0.f, 0.f, 0.f, 0.f};
    if (reducerA) {
        if (wave == 0) {
            own0 = lds_sum(red, lane);
            own1 = lds_sum(red + 2048, lane);
        }
    } else if (wave < 2) {   // wave 0 publishes the gate quads, wave 1 the up quads
        own0 = lds_sum(red + wave * 2048, lane);
    }
    __syncthreads();

    // ---- publish or reduce; every wave but the gathering one requests the weights of its down unit
    // now (the gathering wave's poll results would queue behind them), so that they stream in while the
    // SwiGLU reduction runs ----
    if (!reducerA) {
        if (wave < 2) {
            float *slot = p.partialA + ((size_t)(wave * nprodA + sliceA) * p.tilesA + tileA) * 256 + lane * 2;
            slot_store_planes(slot, 128, keep_sentinel_unique(own0));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (hasB && !gather_wave) load_unit(r0, p.qw[2], p.qz[2], p.sc[2], p.E, tileB, unitB, lg, ln);
    __builtin_amdgcn_sched_barrier(0);
    if (gather_wave) {
        floatx4 g = own0, u = own1;
        floatx4 sg = floatx4{0.f, 0.f, 0.f, 0.f}, su = floatx4{0.f, 0.f, 0.f, 0.f};
        float *base = p.partialA + (size_t)tileA * 256 + lane * 2;
        if (!gather(base, (size_t)p.tilesA * 256, 2 * nprodA, nprodA, sg, su, p.spin_limit))
            __hip_atomic_store(p.header, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        g += sg;
        u += su;
        float out[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float gate = bf16_bits_to_float(float_to_bf16_bits(g[q]));
            const float up = bf16_bits_to_float(float_to_bf16_bits(u[q]));
            out[q] = silu_tanh(gate) * up;
        }
        uint32_t o0 = pack_bf16x2(out[0], out[1]), o1 = pack_bf16x2(out[2], out[3]);
        const int col = tileA * 256 + lane * 4;
        if (p.h_out) *reinterpret_cast<uint2 *>(p.h_out + col) = uint2{o0, o1};
        if (o0 == kEmpty) o0 = 0x7FC07FC0u;   // keep the sentinel unique (both halves NaN either way)
        if (o1 == kEmpty) o1 = 0x7FC07FC0u;
        const uint64_t pair = (uint64_t)o0 | ((uint64_t)o1 << 32);
        for (int t = 0; t < p.tilesB; ++t)
            __hip_atomic_store(reinterpret_cast<uint64_t *>(p.hpriv + (size_t)t * (p.H >> 1) + (col >> 1)), pair,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (hasB) load_unit(r0, p.qw[2], p.qz[2], p.sc[2], p.E, tileB, unitB, lg, ln);
    }

    // ---- down unit: wait for its 128 values of h, take them, hand the chunk back ----
    if (hasB) {
        uint32_t *chunk = p.hpriv + (size_t)tileB * (p.H >> 1) + (size_t)unitB * 64 + 4 * lg;   // + 16 * s words
        int spins = 0;
        for (;;) {
            bool ok = true;
            if (a_valid) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    av[s] = slot_load(reinterpret_cast<const float *>(chunk + 16 * s));
                    ok = ok && slot_full(av[s]);
                }
            }
            if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
            if (++spins > p.spin_limit) {
                if (lane == 0) __hip_atomic_store(p.header, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(POLL_SLEEP);
        }
        if (a_valid) {
#pragma unroll
            for (int s = 0; s < 4; ++s)
                slot_store(reinterpret_cast<float *>(chunk + 16 * s), u32x4{kEmpty, kEmpty, kEmpty, kEmpty});
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) av[s] = u32x4{0u, 0u, 0u, 0u};
        }
        compute_unit(r0, av, yd, nib_mask, magic);
    }

    // ---- down: cross-wave combine, publish or reduce ----
    float *redB = red + 4096;
    lds_put(redB + wave * 256, yd, lg, ln);
    __syncthreads();
    if (wave != 0) return;
    floatx4 own = lds_sum(redB, lane);
    const int nprodB = p.splitB - 1;
    if (!reducerB) {
        slot_store_planes(p.partialB + ((size_t)sliceB * p.tilesB + tileB) * 256 + lane * 2, 128, keep_sentinel_unique(own));
        return;
    }
    floatx4 sum = floatx4{0.f, 0.f, 0.f, 0.f}, unused = floatx4{0.f, 0.f, 0.f, 0.f};
    if (!gather(p.partialB + (size_t)tileB * 256 + lane * 2, (size_t)p.tilesB * 256, nprodB, nprodB, sum, unused, p.spin_limit))
        __hip_atomic_store(p.header, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    floatx4 out = sum + own;
    const int col = tileB * 256 + lane * 4;
    if (p.residual) {
        const uint2 r = *reinterpret_cast<const uint2 *>(p.residual + col);
        out[0] += __builtin_bit_cast(float, r.x << 16);
        out[1] += __builtin_bit_cast(float, r.x & 0xFFFF0000u);
        out[2] += __builtin_bit_cast(float, r.y << 16);
        out[3] += __builtin_bit_cast(float, r.y & 0xFFFF0000u);
    }
    const uint2 o = uint2{pack_bf16x2(out[0], out[1]), pack_bf16x2(out[2], out[3])};
    *reinterpret_cast<uint2 *>(p.y + col) = o;
    if (p.sumsq_out) {   // same expression and order as the streaming kernel's epilogue, so either path feeds the next norm alike
        const float r0 = __builtin_bit_cast(float, o.x << 16), r1 = __builtin_bit_cast(float, o.x & 0xFFFF0000u);
        const float r2 = __builtin_bit_cast(float, o.y << 16), r3 = __builtin_bit_cast(float, o.y & 0xFFFF0000u);
        float sq = fmaf(r0, r0, fmaf(r1, r1, fmaf(r2, r2, r3 * r3)));
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
        if (lane == 0) p.sumsq_out[tileB] = sq;
    }
}

// Shape plan: the largest G <= cus with G = tilesA * splitA = tilesB * splitB, whole units per
// slice, G >= 3/4 of the CUs, at most 8 units per slice (one per wave) and at least 6 (waves mostly busy), at most
// 4 producers per gate/up tile (their 8 slots are one polling batch).
bool plan_ffn_fused(int E, int H, int cus, FfnFusedPlan *pl) {
    if (E <= 0 || H <= 0 || E % 256 || H % 256) return false;
    const int tilesA = H / 256, tilesB = E / 256, unitsA = E / 128, unitsB = H / 128;
    for (int G = cus; 4 * G >= 3 * cus; --G) {   // fewer workgroups than 3/4 of the CUs: two launches fill the chip better
        if (G % tilesA || G % tilesB) continue;
        const int splitA = G / tilesA, splitB = G / tilesB;
        if (unitsA % splitA || unitsB % splitB) continue;
        const int upsA = unitsA / splitA, upsB = unitsB / splitB;
        if (upsA > 8 || upsB > 8 || upsA < 6 || upsB < 6) continue;
        if (splitA < 1 || splitA > 5 || splitB < 1 || splitB > kMaxKSplit) continue;
        *pl = FfnFusedPlan{G, tilesA, splitA, upsA, tilesB, splitB, upsB};
        return true;
    }
    return false;
}

size_t ffn_fused_scratch_bytes(int E, int H, const FfnFusedPlan &pl) {
    const size_t a = (size_t)2 * (pl.splitA - 1) * pl.tilesA * 256 * sizeof(float);
    const size_t b = (size_t)(pl.splitB - 1) * pl.tilesB * 256 * sizeof(float);
    const size_t c = (size_t)pl.tilesB * (H / 2) * sizeof(uint32_t);
    return a + b + c;
}

hipError_t launch_ffn_fused(const FfnFusedPlan &pl, const uint16_t *x, const int32_t *const qw[3], const int32_t *const qz[3],
                            const uint16_t *const sc[3], const uint16_t *residual, uint16_t *y, uint16_t *h_out, int E, int H,
                            void *workspace, hipStream_t stream, const FfnFusedNorm *norm, float *sumsq_out) {
    FfnParams p;
    p.x = x;
    for (int i = 0; i < 3; ++i) {
        p.qw[i] = reinterpret_cast<const uint32_t *>(qw[i]);
        p.qz[i] = reinterpret_cast<const uint32_t *>(qz[i]);
        p.sc[i] = sc[i];
    }
    p.residual = residual;
    p.norm_w = norm ? norm->norm_w : nullptr;
    p.sumsq_in = norm ? norm->sumsq_in : nullptr;
    p.sumsq_n = norm ? norm->sumsq_n : 0;
    p.eps = norm ? norm->eps : 0.f;
    p.y = y;
    p.h_out = h_out;
    p.sumsq_out = sumsq_out;
    p.header = reinterpret_cast<uint32_t *>(workspace);
    char *base = reinterpret_cast<char *>(workspace) + kHeaderBytes;
    p.partialA = reinterpret_cast<float *>(base);
    base += (size_t)2 * (pl.splitA - 1) * pl.tilesA * 256 * sizeof(float);
    p.partialB = reinterpret_cast<float *>(base);
    base += (size_t)(pl.splitB - 1) * pl.tilesB * 256 * sizeof(float);
    p.hpriv = reinterpret_cast<uint32_t *>(base);
    p.E = E;
    p.H = H;
    p.tilesA = pl.tilesA;
    p.splitA = pl.splitA;
    p.upsA = pl.upsA;
    p.tilesB = pl.tilesB;
    p.splitB = pl.splitB;
    p.upsB = pl.upsB;
    p.spin_limit = g_stream_tune.spin_limit > 0 ? g_stream_tune.spin_limit : (1 << 18);
    if (norm)
        hipLaunchKernelGGL(ffn_fused_kernel<true>, dim3(pl.G), dim3(512), 3 * 8 * 256 * sizeof(float), stream, p);
    else
        hipLaunchKernelGGL(ffn_fused_kernel<false>, dim3(pl.G), dim3(512), 3 * 8 * 256 * sizeof(float), stream, p);
    return hipGetLastError();
}

}  // namespace w4a16
