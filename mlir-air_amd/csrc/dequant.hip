// AWQ int4 -> dense bf16 dequant for gfx950.
//
// out[k, n] = bf16_rne((q[k, n] - z[k / 128, n]) * s[k / 128, n]).
// (q - z) and the product are exact in fp32 (5 x 8 significant bits), so the single
// v_cvt_pk_bf16_f32 rounding reproduces the reference bit for bit.
//
// HBM-bound: 0.5 B read + 2 B written per weight.  One thread owns one packed word
// (8 columns) for ROWS consecutive rows of one group: 4-byte loads coalesce to 256 B per
// wavefront and every 16-byte store lands next to its neighbour lane's (1 KiB contiguous
// per wavefront store), which is what the write-dominated traffic needs.
#include "common.h"
#include "kernels.h"

namespace w4a16 {

template <int ROWS>
__global__ void __launch_bounds__(256) dequant_kernel(const uint32_t *__restrict__ qweight,
                                                      const uint32_t *__restrict__ qzeros,
                                                      const uint16_t *__restrict__ scales,
                                                      uint16_t *__restrict__ out, int K, int N) {
    const int nb = N >> 3;
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= nb) return;
    const int k0 = blockIdx.y * ROWS;
    const int g = k0 / kGroup;

    uint32_t w[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) w[i] = __builtin_nontemporal_load(qweight + (size_t)(k0 + i) * nb + b);

    float z[8];
    unpack8_f32(qzeros[(size_t)g * nb + b], z);
    const u32x4 sv = *reinterpret_cast<const u32x4 *>(scales + (size_t)g * N + 8 * b);
    float s[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s[2 * j] = bf16_bits_to_float(sv[j] & 0xFFFFu);
        s[2 * j + 1] = bf16_bits_to_float(sv[j] >> 16);
    }

#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        float q[8];
        unpack8_f32(w[i], q);
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = pack_bf16x2((q[2 * j] - z[2 * j]) * s[2 * j], (q[2 * j + 1] - z[2 * j + 1]) * s[2 * j + 1]);
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(out + (size_t)(k0 + i) * N + 8 * b));
    }
}

// 1-D form on the reference's own tiled buffer (pack_inputs, programming_examples/dequant_awq/dequant_awq.py:259-278):
// `herd_n` tiles of tile_bytes, each [Q: n_tile / 2 bytes, element 2 j in the low nibble of byte j][S: n_tile / gs
// bf16][Z: n_tile / gs u8][pad to 4 bytes].  out[i] = bf16_rne((q[i] - z[i / gs]) * s[i / gs]).  One thread = one
// 4-byte word of nibbles (8 elements, a 16-byte store); a group's scale and zero point are a 2-byte and a 1-byte load.
__global__ void __launch_bounds__(256) dequant_1d_kernel(const uint8_t *__restrict__ packed, uint16_t *__restrict__ out,
                                                         int n_tile, int gs, int tile_bytes, int nwords_total) {
    const int wi = blockIdx.x * 256 + threadIdx.x;   // word index over the whole vector
    if (wi >= nwords_total) return;
    const int words_per_tile = n_tile >> 3;
    const int tile = wi / words_per_tile, w = wi - tile * words_per_tile;
    const uint8_t *t = packed + (size_t)tile * tile_bytes;
    const int q_bytes = n_tile >> 1, ng = n_tile / gs;
    const int g = (w * 8) / gs;
    const uint32_t word = *reinterpret_cast<const uint32_t *>(t + 4 * w);
    const float s = bf16_bits_to_float(*reinterpret_cast<const uint16_t *>(t + q_bytes + 2 * g));
    const float z = static_cast<float>(t[q_bytes + 2 * ng + g]);
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j)   // byte j: elements 2 j (low nibble), 2 j + 1 (high nibble)
        o[j] = pack_bf16x2((nibble_f32(word, 2 * j) - z) * s, (nibble_f32(word, 2 * j + 1) - z) * s);
    *reinterpret_cast<u32x4 *>(out + (size_t)tile * n_tile + 8 * w) = o;
}

hipError_t launch_dequant_1d(const uint8_t *packed, uint16_t *out, int n, int gs, int herd_n, hipStream_t stream) {
    const int n_tile = n / herd_n, ng = n_tile / gs;
    const int tile_bytes = (n_tile / 2 + 3 * ng + 3) & ~3;
    const int nwords = n / 8;
    hipLaunchKernelGGL(dequant_1d_kernel, dim3((nwords + 255) / 256), dim3(256), 0, stream, packed, out, n_tile, gs, tile_bytes,
                       nwords);
    return hipGetLastError();
}

hipError_t launch_dequant(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, uint16_t *out,
                          int K, int N, hipStream_t stream) {
    constexpr int ROWS = 16;
    const int nb = N / 8;
    dim3 grid((nb + 255) / 256, K / ROWS);
    hipLaunchKernelGGL(dequant_kernel<ROWS>, grid, dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t *>(qweight), reinterpret_cast<const uint32_t *>(qzeros),
                       scales, out, K, N);
    return hipGetLastError();
}

}  // namespace w4a16
