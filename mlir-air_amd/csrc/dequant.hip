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
