// Q4NX / Q4_0 block codec for gfx950: dequant to dense bf16 and repack into the operands of the
// streaming kernel's affine path.
//
// One block covers 32 rows (output features) x 256 columns (input features) of W[M, K] and is
// 5120 bytes (programming_examples/fused_decode/proj_qmm_pack.py:4-9):
//     bf16  scales[8 groups][32 rows]        offset    0
//     bf16  mins  [8 groups][32 rows]        offset  512
//     uint8 qs[2 row groups][256 cols][8]    offset 1024   byte kk of (rg, col) = (q[16 rg + 2 kk + 1][col] << 4) | q[16 rg + 2 kk][col]
// A group is 32 consecutive columns of one row.  Blocks are stored row-block major, [M / 32][K / 256].
//
// Three value conventions share the layout (`mode`):
//   0  additive     w = s * q + m, q unsigned       (the proj_qmm kernel, fused_decode/kernels/q4_k.h:9-17)
//   1  subtractive  w = s * (q - m), q unsigned     (bundles with a "Q4NX" header, llms/llama32_1b_q4nx/llama32_1b_q4nx_weights.py:255-261)
//   2  Q4_0         w = s * q, q signed two's complement, mins unused (fused_decode/qwen25_3b_requant.py:13-17)
// All arithmetic is fp32 with one rounding to bf16; s * q is exact in fp32, so mode 0 and 2 round once.
//
// Both kernels are HBM-bound byte shuffles.  In the 8-byte qs entry of (rg, col) the 16 nibbles are
// 16 consecutive rows of one column, i.e. two words of the [K, M / 8] operand the streaming kernel
// reads (8 output features per word), up to the nibble order inside a word.
#include "common.h"
#include "kernels.h"
#include "wstream.h"

namespace w4a16 {

constexpr int kQ4nxRows = 32, kQ4nxCols = 256, kQ4nxGroup = 32, kQ4nxBlockBytes = 5120;

// grid (K / 256, M / 32), 128 threads: thread t owns columns 2t, 2t + 1 of the block for all 32 rows.
// Loads: 2 x 16 B of qs (two columns are adjacent 8-byte entries).  Stores: 4 B per row, 256 B
// contiguous per wavefront.
__global__ void __launch_bounds__(128) q4nx_dequant_kernel(const uint8_t *__restrict__ blocks, uint16_t *__restrict__ out,
                                                           int K, int mode) {
    const int bj = blockIdx.x, bi = blockIdx.y;
    const uint8_t *blk = blocks + ((size_t)bi * gridDim.x + bj) * kQ4nxBlockBytes;
    const int c = 2 * threadIdx.x;
    const int g = c / kQ4nxGroup;
    const uint16_t *sc = reinterpret_cast<const uint16_t *>(blk) + g * kQ4nxRows;
    const uint16_t *mn = reinterpret_cast<const uint16_t *>(blk + 512) + g * kQ4nxRows;
    uint16_t *dst = out + (size_t)bi * kQ4nxRows * K + (size_t)bj * kQ4nxCols + c;
#pragma unroll
    for (int rg = 0; rg < 2; ++rg) {
        const u32x4 qv = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(blk + 1024 + ((size_t)rg * kQ4nxCols + c) * 8));
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = rg * 16 + r;
            // nibble r of the entry: word r / 8, bit position 4 * (r % 8) (byte r / 2, low nibble first)
            uint32_t q0 = (qv[r >> 3] >> (4 * (r & 7))) & 0xFu;
            uint32_t q1 = (qv[2 + (r >> 3)] >> (4 * (r & 7))) & 0xFu;
            const float s = bf16_bits_to_float(sc[row]);
            const float m = bf16_bits_to_float(mn[row]);
            float w0, w1;
            if (mode == 2) {
                w0 = s * (float)((int)(q0 ^ 8u) - 8);
                w1 = s * (float)((int)(q1 ^ 8u) - 8);
            } else if (mode == 1) {
                w0 = s * ((float)q0 - m);
                w1 = s * ((float)q1 - m);
            } else {
                w0 = fmaf(s, (float)q0, m);
                w1 = fmaf(s, (float)q1, m);
            }
            __builtin_nontemporal_store(pack_bf16x2(w0, w1), reinterpret_cast<uint32_t *>(dst + (size_t)row * K));
        }
    }
}

hipError_t launch_q4nx_dequant(const void *blocks, uint16_t *out, int M, int K, int mode, hipStream_t stream) {
    hipLaunchKernelGGL(q4nx_dequant_kernel, dim3(K / kQ4nxCols, M / kQ4nxRows), dim3(128), 0, stream,
                       reinterpret_cast<const uint8_t *>(blocks), out, K, mode);
    return hipGetLastError();
}

// Nibble i (natural: row 8 * word + i) of `w` to the bit position the streaming kernel expects.
__device__ __forceinline__ uint32_t to_pack_order(uint32_t w) {
    uint32_t o = 0;
#pragma unroll
    for (int pos = 0; pos < 8; ++pos) o |= ((w >> (4 * pack_order(pos))) & 0xFu) << (4 * pos);
    return o;
}

// Blocks -> operands of the streaming kernel's affine path, for y = x . W^T with x[*, K]:
//   qweight int32 [K, M / 8]   word (k, j) holds rows 8 j .. 8 j + 7 of column k, unsigned, AWQ nibble order
//   scales, mins bf16 [K / 32, M]   such that w = q * scale + min
// mode 1 stores min' = -s * m (rounded to bf16 once more: one extra rounding, stated in the header);
// mode 2 stores q ^ 8 and min' = -8 s (exact).
// grid (K / 256, M / 32), 256 threads = the block's columns.  Per thread: 16 B of qs in, 4 words
// out at stride M / 8 words; the 64 lanes of a wavefront write 64 consecutive k rows of the same
// 16 bytes (one 16-byte store each), and the block's 512 scale/min values are moved by threads 0..255.
__global__ void __launch_bounds__(256) q4nx_repack_kernel(const uint8_t *__restrict__ blocks, uint32_t *__restrict__ qweight,
                                                          uint16_t *__restrict__ scales, uint16_t *__restrict__ mins, int M,
                                                          int mode) {
    const int bj = blockIdx.x, bi = blockIdx.y;
    const uint8_t *blk = blocks + ((size_t)bi * gridDim.x + bj) * kQ4nxBlockBytes;
    const int col = threadIdx.x;
    const int nb = M >> 3;
    u32x4 o;
#pragma unroll
    for (int rg = 0; rg < 2; ++rg) {
        const uint2 qv = *reinterpret_cast<const uint2 *>(blk + 1024 + ((size_t)rg * kQ4nxCols + col) * 8);
        const uint32_t flip = mode == 2 ? 0x88888888u : 0u;
        o[2 * rg] = to_pack_order(qv.x ^ flip);
        o[2 * rg + 1] = to_pack_order(qv.y ^ flip);
    }
    *reinterpret_cast<u32x4 *>(qweight + ((size_t)bj * kQ4nxCols + col) * nb + bi * 4) = o;

    // scales[g][row] -> [bj * 8 + g][bi * 32 + row]
    const int g = threadIdx.x >> 5, row = threadIdx.x & 31;
    const uint16_t sb = reinterpret_cast<const uint16_t *>(blk)[threadIdx.x];
    const uint16_t mb = reinterpret_cast<const uint16_t *>(blk + 512)[threadIdx.x];
    const float s = bf16_bits_to_float(sb), m = bf16_bits_to_float(mb);
    uint16_t m_out = mb;
    if (mode == 1) m_out = float_to_bf16_bits(-(s * m));
    if (mode == 2) m_out = float_to_bf16_bits(-8.0f * s);
    const size_t dst = ((size_t)bj * 8 + g) * M + bi * kQ4nxRows + row;
    scales[dst] = sb;
    mins[dst] = m_out;
}

hipError_t launch_q4nx_repack(const void *blocks, int32_t *qweight, uint16_t *scales, uint16_t *mins, int M, int K,
                              int mode, hipStream_t stream) {
    hipLaunchKernelGGL(q4nx_repack_kernel, dim3(K / kQ4nxCols, M / kQ4nxRows), dim3(256), 0, stream,
                       reinterpret_cast<const uint8_t *>(blocks), reinterpret_cast<uint32_t *>(qweight), scales, mins, M,
                       mode);
    return hipGetLastError();
}

// Blocks -> Q4NX stream order (wstream.h) in one pass, the form the whole-K decode kernels and the tiled kernel read:
// the counterpart of the reference's single load-time re-pack of the bundle's blocks into the order its cores consume
// (programming_examples/fused_decode/proj_qmm_pack.py:61-140).  Same bytes as q4nx_repack_kernel followed by
// repack_ws_q4_kernel, without the intermediate operands.  One thread per dword of the buffer.
//   cell dword (tile, group g, lane (lg, ln), K-step t): nibble p = q[n = 16 tile + ln][k = 128 g + 32 t + 8 lg + order(p)],
//     i.e. block (tile / 2, g / 2), row group tile % 2, nibble ln of the eight entries of columns
//     128 (g % 2) + 32 t + 8 lg + 0..7: 64 contiguous bytes, shared by the 16 lanes ln
//   scale word (tile, block b, K-step t, lane (lg, ln), dword i): group g = 16 b + 4 lg + i, the block's column group
//     4 (g % 2) + t, row 16 (tile % 2) + ln
__global__ void __launch_bounds__(256) q4nx_blocks_to_stream_kernel(const uint8_t *__restrict__ blocks, uint32_t *__restrict__ out, int G,
                                                                   int NB, int tiles, int KB, int mode) {
    const size_t tile_dwords = (size_t)(kWsQ4MdKiB * NB + G) * (kWsCellBytes / 4);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= tile_dwords * tiles) return;
    const int tile = (int)(idx / tile_dwords);
    const int off = (int)(idx - (size_t)tile * tile_dwords);
    constexpr int BLOCK_DWORDS = (kWsBlockGroups + kWsQ4MdKiB) * (int)(kWsCellBytes / 4);
    const int b = min(off / BLOCK_DWORDS, NB - 1);
    const int within = off - b * BLOCK_DWORDS;
    const int l = (within & 255) >> 2, sub = within & 3;   // lane and dword of a 1 KiB piece
    const int lg = l >> 4, ln = l & 15;
    const int bi = tile >> 1, rg = tile & 1;
    uint32_t v = 0;
    if (within < kWsQ4MdKiB * 256) {
        const int t = within >> 8;
        const int g = kWsBlockGroups * b + 4 * lg + sub;
        if (g < G) {
            const uint8_t *blk = blocks + ((size_t)bi * KB + (g >> 1)) * kQ4nxBlockBytes;
            const int at = (4 * (g & 1) + t) * kQ4nxRows + 16 * rg + ln;
            const uint16_t sb = reinterpret_cast<const uint16_t *>(blk)[at];
            uint16_t mb = reinterpret_cast<const uint16_t *>(blk + 512)[at];
            const float sc = bf16_bits_to_float(sb);
            if (mode == 1) mb = float_to_bf16_bits(-(sc * bf16_bits_to_float(mb)));
            if (mode == 2) mb = float_to_bf16_bits(-8.0f * sc);
            v = (uint32_t)sb | ((uint32_t)mb << 16);
        }
    } else {
        const int g = kWsBlockGroups * b + (within >> 8) - kWsQ4MdKiB;
        const uint8_t *blk = blocks + ((size_t)bi * KB + (g >> 1)) * kQ4nxBlockBytes;
        const int col0 = 128 * (g & 1) + 32 * sub + 8 * lg;
        const uint32_t *qs = reinterpret_cast<const uint32_t *>(blk + 1024 + ((size_t)rg * kQ4nxCols + col0) * 8);
        const uint32_t flip = mode == 2 ? 8u : 0u;
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int c = pack_order(p);                              // column col0 + c: entry c, nibble ln of its 16
            const uint32_t word = qs[2 * c + (ln >> 3)];
            v |= (((word >> (4 * (ln & 7))) & 0xFu) ^ flip) << (4 * p);
        }
    }
    out[idx] = v;
}

hipError_t launch_q4nx_blocks_to_stream(const void *blocks, void *out, int M, int K, int mode, hipStream_t stream) {
    const size_t dwords = ws_q4_matrix_bytes(K, M) / 4;
    const size_t grid = (dwords + 255) / 256;
    hipLaunchKernelGGL(q4nx_blocks_to_stream_kernel, dim3((unsigned)grid), dim3(256), 0, stream, reinterpret_cast<const uint8_t *>(blocks),
                       static_cast<uint32_t *>(out), K / kGroup, ws_blocks(K), M / kWsTileCols, K / kQ4nxCols, mode);
    return hipGetLastError();
}

}  // namespace w4a16
