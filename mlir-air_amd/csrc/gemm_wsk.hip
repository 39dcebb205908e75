// Batched decode on stream-order weights (wstream.h) for 17 <= M <= 64 rows per launch, split along K:
// y[M, N] = bf16(x[M, K] . W (+ residual)), exact weights (q - z) s, fp32 accumulation.
//
// What bounds a batch of this size is the x a compute unit takes in.  A workgroup that owns its columns for all of K
// (gemm_ws_rows_kernel) reads all of x, M K 2 bytes, whatever its width, and with 64-column workgroups that is 512 KB
// beside 143 KB of weights at M = 64, K = 4096.  Here a workgroup owns 256 columns (16 stream tiles, two per wave)
// for one slice of K: the x tile of a group goes through LDS once per workgroup (16 RT rows x 256 bytes, double
// buffered, XOR-swizzled so that the MFMA A operand reads are conflict-free) and feeds all 16 tiles, so the x traffic
// of the launch falls by four and a workgroup takes in as much x as weights.  The slices' fp32 partial sums go to a
// plain scratch buffer and a second small launch adds them in slice order (deterministic) and rounds once; nothing
// is exchanged between workgroups inside a launch.
//
//   workgroup  = 8 waves, column set bx (tiles 16 bx .. 16 bx + 15), K-slice by (groups by * gps .. + gps - 1)
//   wave w     = tiles 16 bx + 2 w, + 1; RT row tiles of 16 rows: acc[RT][2] per group, flushed per group as in the
//                whole-K kernels, y += s (sum (128 + q) x - (128 + z) sum x)
//   sum x      = per (row, group), taken while the x tile is written to LDS (16 lanes hold a row: one DPP row sum)
//   quad       = 4 consecutive groups of a block: their scale words are one 16-byte chunk per (tile, column); the
//                quad's 8 cells and 2 chunks per lane are requested a quad ahead
#include <algorithm>

#include "common.h"
#include "kernels.h"
#include "wstream.h"

namespace w4a16 {

namespace {

constexpr int kSkWaves = 8;
constexpr int kSkSetTiles = 16;    // stream tiles (of 16 columns) per workgroup
constexpr int kSkMaxSlices = 16;

__device__ __forceinline__ bf16x8 sk_cell_operand(uint32_t w, uint32_t nib_mask, uint32_t magic) {
    u32x4 b;
#pragma unroll
    for (int v = 0; v < 4; ++v) b[v] = ((w >> (4 * v)) & nib_mask) | magic;   // rows (2 v, 2 v + 1) as bf16 (128 + q)
    return __builtin_bit_cast(bf16x8, b);
}

template <int RT>
__global__ void __launch_bounds__(kSkWaves * 64) gemm_wsk_kernel(const uint16_t *__restrict__ x, const char *__restrict__ w,
                                                                 float *__restrict__ partial, uint16_t *__restrict__ y,
                                                                 const uint16_t *__restrict__ residual, int M, int K, int N, int G,
                                                                 int NB, int gps) {
    constexpr int ROWS = 16 * RT, XT = ROWS * 256;        // rows and bytes of an x tile (one group: 128 bf16 per row)
    constexpr int XL = (ROWS * 16) / (kSkWaves * 64);     // 16-byte chunks of a tile per thread (RT = 2: 1, RT = 4: 2)
    static_assert(RT == 2 || RT == 4, "row tiles per launch");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // [2][ROWS][256 B], then [2][ROWS] row sums
    float *xs_lds = reinterpret_cast<float *>(lds + 2 * XT);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    const int g_lo = blockIdx.y * gps, g_hi = min(G, g_lo + gps);   // (the host launches no empty slice)
    const int ntiles = N / kWsTileCols;
    const int tile0 = blockIdx.x * kSkSetTiles + 2 * wave;
    const bool have0 = tile0 < ntiles, have1 = tile0 + 1 < ntiles;
    const size_t tile_bytes = (size_t)(NB + G) * kWsCellBytes;
    // a wave without a tile (ragged last set) reads the last tile's bytes and stores nothing
    const char *tb0 = w + (size_t)(have0 ? tile0 : ntiles - 1) * tile_bytes;
    const char *tb1 = w + (size_t)(have1 ? tile0 + 1 : ntiles - 1) * tile_bytes;

    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));

    floatx4 Y[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) Y[rt][0] = Y[rt][1] = floatx4{0.f, 0.f, 0.f, 0.f};

    // ---- x tile: global -> registers -> LDS ----
    u32x4 xr[XL];
    auto load_x = [&](int g) {
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int idx = tid + kSkWaves * 64 * j, row = idx >> 4, chunk = idx & 15;
            // (requested as it is, a row past M as row M - 1, and zeroed when the registers go to LDS: a select here would
            // make the wave wait for the request on the spot, and for every older request with it)
            xr[j] = *reinterpret_cast<const u32x4 *>(x + (size_t)min(row, M - 1) * K + (size_t)g * kGroup + chunk * 8);
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int j = 0; j < XL; ++j) {
            const int idx = tid + kSkWaves * 64 * j, row = idx >> 4, chunk = idx & 15;
            const u32x4 v = row < M ? xr[j] : u32x4{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4 *>(lds + buf * XT + row * 256 + ((chunk ^ (row & 15)) << 4)) = v;
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                s += __builtin_bit_cast(float, v[e] << 16) + __builtin_bit_cast(float, v[e] & 0xFFFF0000u);
            s = row_sum16(s);   // the 16 lanes of a DPP row hold the 16 chunks of one x row
            if (chunk == 0) xs_lds[buf * ROWS + row] = s;
        }
    };

    // ---- weights of a quad (4 groups of one block): 8 cells and, per tile, the chunk of 4 scale words ----
    struct Quad {
        u32x4 cell[4][2];
        u32x4 md;   // lane (lg, ln): the chunk of tile lg & 1, column ln
    };
    auto load_quad = [&](int gq, Quad &q) {
        const int b = gq >> 4, gl = gq & 15;
        const size_t blk = (size_t)b * ((kWsBlockGroups + 1) * kWsCellBytes);
        q.md = *reinterpret_cast<const u32x4 *>(((lg & 1) ? tb1 : tb0) + blk + (size_t)(16 * (gl >> 2) + ln) * 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gj = gq + j < G ? gl + j : gl;   // (past the end of K: re-read a cell in range, never used)
            q.cell[j][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(tb0 + blk + (size_t)(1 + gj) * kWsCellBytes) + lane);
            q.cell[j][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(tb1 + blk + (size_t)(1 + gj) * kWsCellBytes) + lane);
        }
    };

    Quad cur, nxt;
    load_x(g_lo);
    load_quad(g_lo, cur);
    store_x(0);
    __syncthreads();

    int buf = 0;
    for (int gq = g_lo; gq < g_hi; gq += 4) {
        // (the x tile of the next group first: the wait for it then leaves the younger requests, the next quad's cells, in flight)
        if (gq + 1 < g_hi) load_x(gq + 1);
        __builtin_amdgcn_sched_barrier(0);
        if (gq + 4 < g_hi) load_quad(gq + 4, nxt);
        // the chunk of the other tile sits in the lane 16 away
        u32x4 other;
#pragma unroll
        for (int e = 0; e < 4; ++e) other[e] = (uint32_t)__shfl_xor((int)cur.md[e], 16);
        const u32x4 md0 = (lg & 1) ? other : cur.md, md1 = (lg & 1) ? cur.md : other;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int g = gq + j;
            if (g >= g_hi) break;   // workgroup-uniform
            const bool more = g + 1 < g_hi;
            if (more && j > 0) load_x(g + 1);
            floatx4 acc[RT][2];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) acc[rt][0] = acc[rt][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                bf16x8 a[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    a[rt] = *reinterpret_cast<const bf16x8 *>(lds + buf * XT + (16 * rt + ln) * 256 + (((4 * t + lg) ^ ln) << 4));
                const bf16x8 b0 = sk_cell_operand(cur.cell[j][0][t], nib_mask, magic);
                const bf16x8 b1 = sk_cell_operand(cur.cell[j][1][t], nib_mask, magic);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b0, acc[rt][0], 0, 0, 0);
                    acc[rt][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b1, acc[rt][1], 0, 0, 0);
                }
            }
            // group flush: register i of lane group lg is row 16 rt + 4 lg + i
            const float s0 = __builtin_bit_cast(float, md0[j] << 16), nz0 = __builtin_bit_cast(float, md0[j] & 0xFFFF0000u);
            const float s1 = __builtin_bit_cast(float, md1[j] << 16), nz1 = __builtin_bit_cast(float, md1[j] & 0xFFFF0000u);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const floatx4 xs = *reinterpret_cast<const floatx4 *>(xs_lds + buf * ROWS + 16 * rt + 4 * lg);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    Y[rt][0][i] = fmaf(s0, fmaf(nz0, xs[i], acc[rt][0][i]), Y[rt][0][i]);
                    Y[rt][1][i] = fmaf(s1, fmaf(nz1, xs[i], acc[rt][1][i]), Y[rt][1][i]);
                }
            }
            if (more) store_x(buf ^ 1);   // (that stage was last read a group ago, before the barrier below)
            __syncthreads();
            buf ^= 1;
        }
        if (gq + 4 < g_hi) cur = nxt;
    }

    // ---- this slice's sums: to the scratch buffer, or (one slice) straight to y ----
    const int slices = gridDim.y;
    if (slices > 1) {
        // Through LDS, so that a wave stores whole rows of the workgroup's 256 columns (1 KiB per instruction) instead
        // of four 64-byte pieces: rows padded by 4 floats, which spreads the four lane groups (4 rows apart) over all banks.
        constexpr int LDP = 16 * kSkSetTiles + 4;
        float *yt = reinterpret_cast<float *>(lds);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int i = 0; i < 4; ++i) yt[(16 * rt + 4 * lg + i) * LDP + (2 * wave + c) * kWsTileCols + ln] = Y[rt][c][i];
        __syncthreads();
        const int col0 = blockIdx.x * kSkSetTiles * kWsTileCols, ncols = min(kSkSetTiles * kWsTileCols, N - col0);   // a multiple of 16
        float *dst = partial + (size_t)blockIdx.y * M * N + col0;
        for (int row = wave; row < M; row += kSkWaves)
            if (4 * lane < ncols)
                *reinterpret_cast<floatx4 *>(dst + (size_t)row * N + 4 * lane) = *reinterpret_cast<const floatx4 *>(yt + row * LDP + 4 * lane);
        return;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            if (!(c ? have1 : have0)) continue;
            const int col = (tile0 + c) * kWsTileCols + ln;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 16 * rt + 4 * lg + i;
                if (row >= M) continue;
                const size_t at = (size_t)row * N + col;
                if (slices > 1) {
                    partial[(size_t)blockIdx.y * M * N + at] = Y[rt][c][i];
                } else {
                    float v = Y[rt][c][i];
                    if (residual) v += bf16_bits_to_float(residual[at]);
                    y[at] = float_to_bf16_bits(v);
                }
            }
        }
}

// y = bf16(sum over the slices, in slice order (+ residual)); four columns per thread
__global__ void __launch_bounds__(256) gemm_wsk_reduce_kernel(const float *__restrict__ partial, const uint16_t *__restrict__ residual,
                                                              uint16_t *__restrict__ y, size_t mn, int slices) {
    const size_t at = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (at >= mn) return;
    floatx4 s = *reinterpret_cast<const floatx4 *>(partial + at);
    for (int k = 1; k < slices; ++k) {
        const floatx4 v = *reinterpret_cast<const floatx4 *>(partial + (size_t)k * mn + at);
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] += v[i];
    }
    if (residual) {
        const uint2 r = *reinterpret_cast<const uint2 *>(residual + at);
        s[0] += bf16_bits_to_float(r.x & 0xFFFFu), s[1] += bf16_bits_to_float(r.x >> 16);
        s[2] += bf16_bits_to_float(r.y & 0xFFFFu), s[3] += bf16_bits_to_float(r.y >> 16);
    }
    *reinterpret_cast<uint2 *>(y + at) = uint2{pack_bf16x2(s[0], s[1]), pack_bf16x2(s[2], s[3])};
}

// Slices of K for `rows` rows: enough workgroups for the chip (column sets x slices >= ~256), whole quads of groups
// per slice, at most kSkMaxSlices.
int sk_slices(int K, int N, int *gps_out) {
    const int G = K / kGroup, sets = (N / kWsTileCols + kSkSetTiles - 1) / kSkSetTiles;
    int want = (256 + sets - 1) / sets;
    if (want > kSkMaxSlices) want = kSkMaxSlices;
    if (want < 1) want = 1;
    int gps = ((G + want - 1) / want + 3) & ~3;   // groups per slice: a multiple of 4
    if (gps < 4) gps = 4;
    *gps_out = gps;
    return (G + gps - 1) / gps;
}

}  // namespace

// Where the split pays, measured against the whole-K launches (gemm_ws_rows_kernel) at K 2048 .. 14336, N 2048 .. 14336
// and 17 .. 128 rows: the whole-K launches re-read the x rows once per 16, 32 or 64 columns, so they lose with long K,
// many rows and narrow workgroups (K = 4096, N = 6144, 64 rows: 34.2 us whole-K, 18.1 us split; K = 14336, N = 4096,
// 64 rows: 59.0 / 27.9), and win where the split has only a few groups per slice to spread its fixed costs over (the
// second launch, the x tile through LDS: K = 2048, N = 8192: 12.6 / 14.6 us at 64 rows) or where their workgroups are 64
// columns wide already (N >= 12800: K = 4096, N = 14336, 64 rows: 24.5 / 26.1 us).
bool gemm_wsk_pays(int M, int K, int N) {
    if (g_gemv_ws_tune.splitk) return g_gemv_ws_tune.splitk == 1;
    const int G = K / kGroup, tiles = N / kWsTileCols, rows = M < 64 ? M : 64;
    const bool wide_whole_k = tiles % 4 == 0 && tiles / 4 >= 200;   // launch_gemm_ws takes 64-column workgroups there
    return G >= 32 && rows * G >= 1536 && !wide_whole_k;
}

size_t gemm_wsk_scratch_bytes(int M, int K, int N) {
    int gps = 0;
    const int slices = sk_slices(K, N, &gps);
    const int rows = M < 64 ? M : 64;
    return slices > 1 ? (size_t)slices * rows * N * sizeof(float) : 0;
}

// Launches of up to 64 rows.  `scratch`: gemm_wsk_scratch_bytes(M, K, N) bytes of plain scratch (no initialisation, nothing
// kept), may be null when that is 0.
hipError_t launch_gemm_wsk(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, float *scratch, int M, int K,
                           int N, hipStream_t stream) {
    const int G = K / kGroup, NB = ws_blocks(K);
    int gps = 0;
    const int slices = sk_slices(K, N, &gps);
    if (slices > 1 && !scratch) return hipErrorInvalidValue;
    const int sets = (N / kWsTileCols + kSkSetTiles - 1) / kSkSetTiles;
    for (int m0 = 0; m0 < M; m0 += 64) {
        const int rows = M - m0 < 64 ? M - m0 : 64;
        const uint16_t *xr = x + (size_t)m0 * K, *rr = residual ? residual + (size_t)m0 * N : nullptr;
        uint16_t *yr = y + (size_t)m0 * N;
        const dim3 grid(sets, slices), block(kSkWaves * 64);
        if (rows > 32) {
            const size_t lds = std::max<size_t>(2 * (size_t)64 * 256 + 2 * 64 * sizeof(float), (size_t)64 * (16 * kSkSetTiles + 4) * sizeof(float));
            hipError_t ea = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_wsk_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (ea != hipSuccess) return ea;
            hipLaunchKernelGGL((gemm_wsk_kernel<4>), grid, block, lds, stream, xr, static_cast<const char *>(w), scratch, yr, rr, rows, K, N,
                               G, NB, gps);
        } else {
            const size_t lds = std::max<size_t>(2 * (size_t)32 * 256 + 2 * 32 * sizeof(float), (size_t)32 * (16 * kSkSetTiles + 4) * sizeof(float));
            hipLaunchKernelGGL((gemm_wsk_kernel<2>), grid, block, lds, stream, xr, static_cast<const char *>(w), scratch, yr, rr, rows, K, N,
                               G, NB, gps);
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (slices > 1) {
            const size_t mn = (size_t)rows * N;   // N % 16 == 0: whole groups of four columns
            hipLaunchKernelGGL(gemm_wsk_reduce_kernel, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, stream, scratch, rr, yr, mn,
                               slices);
            e = hipGetLastError();
            if (e != hipSuccess) return e;
        }
    }
    return hipSuccess;
}

}  // namespace w4a16
