// Prefill W4A16 GEMM for gfx950: y[M, N] = bf16(x[M, K] . W), M > 16.
//
// Compute-bound.  Each workgroup owns a BM x BN output tile and walks K in steps of BK.
// Per step the x tile is copied to LDS and the packed weight tile is dequantised ONCE to
// bf16 - bit-identical to the dense dequant kernel, W = bf16_rne((q - z) * s) - and written
// to LDS in [n][k] order, so both MFMA operands are 16-byte ds_read_b128 of 8 consecutive k.
// v_mfma_f32_32x32x16_bf16 accumulates in fp32; one bf16 rounding at the end.
//
// Dequant work is shared by the whole M-tile: a thread takes the same packed word from 4
// consecutive rows (same 8 columns), so each column's 4 k-values leave as one ds_write_b64.
#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDK = BK + 8;   // padded LDS row (bf16 elements): 144 B keeps ds_read_b128 conflict-free
constexpr int kThreads = 256;

struct GemmParams {
    const uint16_t *x;
    const uint32_t *qw;
    const uint32_t *qz;
    const uint16_t *sc;
    uint16_t *y;
    int M, K, N;
    int tiles_m, tiles_n;
};

__global__ void __launch_bounds__(kThreads) gemm_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t sA[BM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t sB[BN * LDK];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;   // 2 x 2 waves, 64 x 64 each

    // Each XCD (blockIdx % 8) walks a contiguous range of tiles, M fastest, so the
    // workgroups sharing an L2 reuse the same weight tile across their M tiles.
    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int tile = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (tile >= total) return;
    const int tm = tile % p.tiles_m, tn = tile / p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const int nb = p.N >> 3;

    // ---- global -> register staging assignments ----
    // A: 128 rows x 64 k = 1024 x 16 B; thread takes 4 pieces: row = tid / 8 + 32 * i, kseg = tid % 8.
    const int a_row = tid >> 3, a_seg = tid & 7;
    // B: item = (octet of rows, word column); two threads per item (4 rows each).
    const int b_col = tid & 15;          // word column inside the tile (8 columns)
    const int b_quad = tid >> 4;         // 0..15: rows 4 * b_quad .. +3 of the K tile
    int b_word = (n0 >> 3) + b_col;
    if (b_word >= nb) b_word = nb - 1;   // ragged N: load in range, never stored

    u32x4 ra[4];
    uint32_t rb[4];
    uint32_t rz;
    u32x4 rs;

    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int row = m0 + a_row + 32 * i;
            if (row >= p.M) row = p.M - 1;
            ra[i] = *reinterpret_cast<const u32x4 *>(p.x + (size_t)row * p.K + k0 + 8 * a_seg);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) rb[i] = p.qw[(size_t)(k0 + 4 * b_quad + i) * nb + b_word];
        const int g = k0 / kGroup;
        rz = p.qz[(size_t)g * nb + b_word];
        rs = *reinterpret_cast<const u32x4 *>(p.sc + (size_t)g * p.N + 8 * (size_t)b_word);
    };

    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<u32x4 *>(&sA[(a_row + 32 * i) * LDK + 8 * a_seg]) = ra[i];
        float z[8], s[8], q[4][8];
        unpack8_f32(rz, z);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s[2 * j] = bf16_bits_to_float(rs[j] & 0xFFFFu);
            s[2 * j + 1] = bf16_bits_to_float(rs[j] >> 16);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) unpack8_f32(rb[i], q[i]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint2 v;
            v.x = pack_bf16x2((q[0][j] - z[j]) * s[j], (q[1][j] - z[j]) * s[j]);
            v.y = pack_bf16x2((q[2][j] - z[j]) * s[j], (q[3][j] - z[j]) * s[j]);
            *reinterpret_cast<uint2 *>(&sB[(8 * b_col + j) * LDK + 4 * b_quad]) = v;
        }
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int frag_row = lane & 31;        // row (A) / column (B) inside a 32-wide MFMA tile
    const int frag_k = 8 * (lane >> 5);    // k offset inside a 16-wide MFMA step

    load_tile(0);
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        store_tile();
        __syncthreads();
        if (k0 + BK < p.K) load_tile(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = *reinterpret_cast<const bf16x8 *>(&sA[(wm * 64 + i * 32 + frag_row) * LDK + kk + frag_k]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j] = *reinterpret_cast<const bf16x8 *>(&sB[(wn * 64 + j * 32 + frag_row) * LDK + kk + frag_k]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // D layout of the 32x32 MFMA: register r of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < p.M && col < p.N) p.y[(size_t)row * p.N + col] = float_to_bf16_bits(acc[i][j][r]);
            }
        }
}

}  // namespace

hipError_t launch_gemm_prefill(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                               const uint16_t *scales, uint16_t *y, int M, int K, int N, hipStream_t stream) {
    GemmParams p;
    p.x = x;
    p.qw = reinterpret_cast<const uint32_t *>(qweight);
    p.qz = reinterpret_cast<const uint32_t *>(qzeros);
    p.sc = scales;
    p.y = y;
    p.M = M;
    p.K = K;
    p.N = N;
    p.tiles_m = (M + BM - 1) / BM;
    p.tiles_n = (N + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(gemm_kernel, dim3(grid), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
}

}  // namespace w4a16
