// Split-K streaming W4A16 kernel for M <= 16 (decode GEMV, batched decode, SwiGLU front half).
//
// HBM-bound: every packed weight byte is read exactly once with 16-byte loads.  The
// arithmetic runs on the matrix cores even at M = 1, because the fp32 VALU cannot keep
// up with HBM: at 8 TB/s the chip has ~2.5 VALU lane-ops per weight, and a convert + FMA
// path needs ~2.4.  Building MFMA operands costs ~1 op per weight and the MACs are free.
//
// Work decomposition
//   tile   = 512 output columns = 16 lanes x one 16-byte chunk (32 columns) per lane
//   K-step = 32 rows = one v_mfma_f32_16x16x32_bf16; lane (lg, ln) = (lane / 16, lane % 16)
//            loads rows 8*lg .. 8*lg+7 of chunk ln, i.e. exactly the K-slice the MFMA B
//            operand wants from that lane.  One load instruction covers 4 x 256 B segments.
//   unit   = KSTEPS consecutive K-steps inside one quantisation group, loaded up front
//   wave   = `units` units; workgroup = WAVES waves on one (tile, K-slice); the grid is
//            (tiles x ksplit) with all K-slices of a tile on the same XCD.
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
// Cross-wave combine goes through LDS, the cross-workgroup combine through fp32 partials in
// the workspace; the last workgroup to arrive at a tile (arrival counter) sums the partials
// in fixed order (deterministic), applies the epilogue and resets the counter.
#include "common.h"
#include "kernels.h"

namespace w4a16 {

StreamTune g_stream_tune;

struct StreamParams {
    const uint16_t *x;
    const u32x4 *qw[2];
    const u32x4 *qz[2];
    const uint16_t *sc[2];
    uint16_t *y;
    float *partial;
    uint32_t *counters;
    int M, K, N;
    int nchunks;   // N / 32
    int ntiles;    // ceil(nchunks / 16)
    int ksplit;    // workgroups along K per tile
    int units;     // units per wave
    int nmat;      // 1, or 2 for gate/up with the SwiGLU epilogue
    int slots;     // LDS combine slots (power of two, divides WAVES)
};

constexpr int kTileCols = 512;
constexpr int kRowStride = 32 * 17;   // LDS floats per output row: [j (32)][ln (16) + 1 pad]

__device__ __forceinline__ float silu_tanh(float g) { return g * 0.5f * (tanhf(g * 0.5f) + 1.0f); }

template <int KSTEPS, int WAVES, int MI>
__global__ void __launch_bounds__(WAVES * 64) stream_kernel(const StreamParams p) {
    extern __shared__ float red[];
    __shared__ int s_last;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int lg = lane >> 4;
    const int ln = lane & 15;

    // blockIdx -> (tile, matrix, K-slice); consecutive block ids go to consecutive XCDs, so
    // the workgroups that share a tile (and its counter and partials) share one L2.
    const int per_tile = p.nmat * p.ksplit;
    const int xcd = blockIdx.x & 7;
    const int local = blockIdx.x >> 3;
    const int tile = (local / per_tile) * 8 + xcd;
    if (tile >= p.ntiles) return;
    const int sub = local % per_tile;
    const int mat = sub / p.ksplit;
    const int kslice = sub % p.ksplit;

    const int chunk = tile * 16 + ln;
    const int chunk_c = chunk < p.nchunks ? chunk : p.nchunks - 1;   // ragged tile: load in range, never written
    const u32x4 *__restrict__ qw = p.qw[mat];
    const u32x4 *__restrict__ qz = p.qz[mat];
    const uint16_t *__restrict__ sc = p.sc[mat];

    // x row held by this lane in the MFMA A operand (A row = ln): m = ln / 4 + 4 * (ln % 4).
    const int am = (ln >> 2) + 4 * (ln & 3);
    const bool a_valid = ((ln & 3) < MI) && (am < p.M);
    const uint16_t *xrow = p.x + (size_t)(a_valid ? am : 0) * p.K + 8 * lg;

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);

    floatx4 yacc[32];
#pragma unroll
    for (int t = 0; t < 32; ++t) yacc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int nksteps = p.K >> 5;
    for (int u = 0; u < p.units; ++u) {
        const int kstep0 = ((kslice * p.units + u) * WAVES + wave) * KSTEPS;
        if (kstep0 >= nksteps) break;   // wave-uniform
        const int g = kstep0 >> 2;

        u32x4 w[KSTEPS][8];
        u32x4 av[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const size_t row0 = (size_t)(kstep0 + s) * 32 + 8 * lg;
#pragma unroll
            for (int i = 0; i < 8; ++i) w[s][i] = __builtin_nontemporal_load(qw + (row0 + i) * p.nchunks + chunk_c);
            av[s] = *reinterpret_cast<const u32x4 *>(xrow + (size_t)(kstep0 + s) * 32);
            if (!a_valid) av[s] = u32x4{0u, 0u, 0u, 0u};
        }
        const u32x4 zw = qz[(size_t)g * p.nchunks + chunk_c];
        u32x4 sv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            sv[q] = *reinterpret_cast<const u32x4 *>(sc + (size_t)g * p.N + (size_t)chunk_c * 32 + 8 * q);

        floatx4 acc[32];
#pragma unroll
        for (int t = 0; t < 32; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
        floatx4 xs = floatx4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, av[s]);
            xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ones, xs, 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t sel = 0x0C000C00u | ((4u + b) << 16) | (uint32_t)b;
                    u32x4 lo, hi;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const uint32_t pr = __builtin_amdgcn_perm(w[s][2 * v + 1][c], w[s][2 * v][c], sel);
                        lo[v] = (pr & 0x000F000Fu) | 0x43004300u;
                        hi[v] = ((pr >> 4) & 0x000F000Fu) | 0x43004300u;
                    }
                    const int t = (c * 4 + b) * 2;
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, lo), acc[t], 0, 0, 0);
                    acc[t + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, hi), acc[t + 1], 0, 0, 0);
                }
            }
        }

        // Group flush: tile t = (word c, nibble position pos = 2b + h) is natural column
        // j = 8c + pack_order(pos) of this lane's chunk.
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int pos = 0; pos < 8; ++pos) {
                const int t = c * 8 + pos;
                const int j = 8 * c + pack_order(pos);
                const float zc = 128.0f + static_cast<float>((zw[c] >> (4 * pos)) & 0xFu);
                const uint32_t sw = sv[j >> 3][(j & 7) >> 1];
                const float sj = bf16_bits_to_float((j & 1) ? (sw >> 16) : (sw & 0xFFFFu));
#pragma unroll
                for (int i = 0; i < MI; ++i) yacc[t][i] = fmaf(sj, fmaf(-zc, xs[i], acc[t][i]), yacc[t][i]);
            }
        }
    }

    // ---- cross-wave combine in LDS: red[slot][m][j * 17 + ln] ----
    const int slot_stride = p.M * kRowStride;
    const int rounds = WAVES / p.slots;
    for (int r = 0; r < rounds; ++r) {
        if (wave / p.slots == r) {
            float *dst = red + (wave % p.slots) * slot_stride;
#pragma unroll
            for (int t = 0; t < 32; ++t) {
                const int j = 8 * (t >> 3) + pack_order(t & 7);
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    const int m = lg + 4 * i;
                    if (m < p.M) {
                        float *q = dst + m * kRowStride + j * 17 + ln;
                        *q = (r == 0) ? yacc[t][i] : (*q + yacc[t][i]);
                    }
                }
            }
        }
        __syncthreads();
    }

    const bool direct = (per_tile == 1);
    const int nelem = p.M * kTileCols;
    const int col0 = tile * kTileCols;
    for (int e = threadIdx.x; e < nelem; e += WAVES * 64) {
        const int m = e >> 9;
        const int col = e & (kTileCols - 1);
        const int gcol = col0 + col;
        if (gcol >= p.N) continue;
        const float *src = red + m * kRowStride + (col & 31) * 17 + (col >> 5);
        float v = 0.f;
        for (int s = 0; s < p.slots; ++s) v += src[s * slot_stride];
        if (direct)
            p.y[(size_t)m * p.N + gcol] = float_to_bf16_bits(v);
        else
            store_agent(p.partial + ((size_t)(mat * p.ksplit + kslice) * p.M + m) * p.N + gcol, v);
    }
    if (direct) return;

    // ---- cross-workgroup combine: last arrival at this tile reduces the partials ----
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(p.counters + tile, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == (uint32_t)per_tile - 1u);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    for (int e = threadIdx.x; e < nelem; e += WAVES * 64) {
        const int m = e >> 9;
        const int gcol = col0 + (e & (kTileCols - 1));
        if (gcol >= p.N) continue;
        float v0 = 0.f;
        for (int ks = 0; ks < p.ksplit; ++ks) v0 += load_agent(p.partial + ((size_t)ks * p.M + m) * p.N + gcol);
        if (p.nmat == 1) {
            p.y[(size_t)m * p.N + gcol] = float_to_bf16_bits(v0);
        } else {
            float v1 = 0.f;
            for (int ks = 0; ks < p.ksplit; ++ks)
                v1 += load_agent(p.partial + ((size_t)(p.ksplit + ks) * p.M + m) * p.N + gcol);
            const float gate = bf16_bits_to_float(float_to_bf16_bits(v0));
            const float up = bf16_bits_to_float(float_to_bf16_bits(v1));
            p.y[(size_t)m * p.N + gcol] = float_to_bf16_bits(silu_tanh(gate) * up);
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(p.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Launch shape: enough workgroups to cover 256 CUs a few times over, with every wave's
// loads issued up front; K-split bounded so the fp32 partials stay a small fraction of
// the weight bytes.
StreamPlan plan_stream(int M, int K, int N) {
    StreamPlan pl;
    pl.mi = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
    pl.ntiles = (N / 32 + 15) / 16;
    const int nksteps = K / 32;
    pl.ksteps = M <= 4 ? 1 : 4;
    pl.waves = 8;
    pl.units = 1;
    if (g_stream_tune.ksteps) pl.ksteps = g_stream_tune.ksteps;
    if (g_stream_tune.waves) pl.waves = g_stream_tune.waves;
    if (g_stream_tune.units) pl.units = g_stream_tune.units;
    // 512-thread workgroups cap a wave at 256 VGPRs; the wide variants need more.
    if (pl.waves == 8 && (pl.ksteps == 4 || pl.mi == 4)) pl.waves = 4;
    auto split = [&]() { return (nksteps + pl.ksteps * pl.waves * pl.units - 1) / (pl.ksteps * pl.waves * pl.units); };
    pl.ksplit = split();
    while (pl.ksplit > kMaxKSplit) {
        pl.units *= 2;
        pl.ksplit = split();
    }
    return pl;
}

template <int KSTEPS, int WAVES, int MI>
static hipError_t launch_one(const StreamParams &p, int grid, size_t lds, hipStream_t stream) {
    hipLaunchKernelGGL((stream_kernel<KSTEPS, WAVES, MI>), dim3(grid), dim3(WAVES * 64), lds, stream, p);
    return hipGetLastError();
}

template <int KSTEPS, int WAVES>
static hipError_t launch_mi(int mi, const StreamParams &p, int grid, size_t lds, hipStream_t stream) {
    switch (mi) {
        case 1: return launch_one<KSTEPS, WAVES, 1>(p, grid, lds, stream);
        case 2: return launch_one<KSTEPS, WAVES, 2>(p, grid, lds, stream);
        default: return launch_one<KSTEPS, WAVES, 4>(p, grid, lds, stream);
    }
}

template <int KSTEPS>
static hipError_t launch_waves(int waves, int mi, const StreamParams &p, int grid, size_t lds, hipStream_t stream) {
    return waves == 4 ? launch_mi<KSTEPS, 4>(mi, p, grid, lds, stream) : launch_mi<KSTEPS, 8>(mi, p, grid, lds, stream);
}

hipError_t launch_stream(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                         const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                         uint16_t *y, int M, int K, int N, void *workspace, hipStream_t stream) {
    const StreamPlan pl = plan_stream(M, K, N);
    StreamParams p;
    p.x = x;
    p.qw[0] = reinterpret_cast<const u32x4 *>(qweight);
    p.qz[0] = reinterpret_cast<const u32x4 *>(qzeros);
    p.sc[0] = scales;
    p.nmat = up_qweight ? 2 : 1;
    p.qw[1] = reinterpret_cast<const u32x4 *>(up_qweight ? up_qweight : qweight);
    p.qz[1] = reinterpret_cast<const u32x4 *>(up_qzeros ? up_qzeros : qzeros);
    p.sc[1] = up_scales ? up_scales : scales;
    p.y = y;
    p.counters = reinterpret_cast<uint32_t *>(workspace);
    p.partial = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + kCounterBytes);
    p.M = M;
    p.K = K;
    p.N = N;
    p.nchunks = N / 32;
    p.ntiles = pl.ntiles;
    p.ksplit = pl.ksplit;
    p.units = pl.units;
    // LDS slots: as many as fit in 64 KiB, power of two, at most one per wave.
    int slots = pl.waves;
    while (slots > 1 && (size_t)slots * M * kRowStride * sizeof(float) > 65536) slots >>= 1;
    p.slots = slots;
    const size_t lds = (size_t)slots * M * kRowStride * sizeof(float);
    const int grid = ((pl.ntiles + 7) / 8) * 8 * p.nmat * pl.ksplit;
    switch (pl.ksteps) {
        case 1: return launch_waves<1>(pl.waves, pl.mi, p, grid, lds, stream);
        case 2: return launch_waves<2>(pl.waves, pl.mi, p, grid, lds, stream);
        default: return launch_waves<4>(pl.waves, pl.mi, p, grid, lds, stream);
    }
}

__global__ void fill_zero_kernel(uint32_t *p, size_t nwords) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nwords; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

hipError_t launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream) {
    const size_t nwords = bytes / 4;
    int grid = (int)((nwords + 255) / 256);
    if (grid > 2048) grid = 2048;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<uint32_t *>(ptr), nwords);
    return hipGetLastError();
}

}  // namespace w4a16
