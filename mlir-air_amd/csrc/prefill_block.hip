// Prefill O projection + FFN block for gfx950: the int4 sibling of the reference's 8-launch prefill ELF
// (programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_ffn_int4_multi.py:4-17, CPU
// reference :644-665) as five launches:
//   1. res1    = bf16(bf16(attn_out . Wo) + x_residual)          GEMM, residual epilogue
//   2. normed2 = bf16((res1 / sqrt(mean(res1^2) + eps)) * w)     rmsnorm_rows_kernel, fp32 per row
//   3. gate    = bf16(normed2 . Wgate)                           GEMM
//   4. h       = bf16(silu(gate) * bf16(normed2 . Wup))          GEMM, SwiGLU epilogue (silu(g) = g / (1 + exp(-g)))
//   5. y       = bf16(bf16(h . Wdown) + res1)                    GEMM, residual epilogue
// A GEMM whose 256 x 256 tiles number less than half the CUs (the O and down projections at the 1B
// model's width) runs split along K, and a small kernel sums the fp32 slices and applies the epilogue.
// The reference's separate add, SwiGLU and up-projection outputs never reach HBM on their own.
#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

constexpr int kNormThreads = 256;
constexpr int kNormChunks = 4;   // 16-byte chunks a thread keeps in registers: K <= 8 * 256 * 4 = 8192

// One workgroup per row; x is read once (chunks stay in registers between the two passes).
__global__ void __launch_bounds__(kNormThreads) rmsnorm_rows_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ w,
                                                                    uint16_t *__restrict__ out, int K, float eps) {
    __shared__ float part[kNormThreads / 64];
    const int t = threadIdx.x;
    const size_t row = blockIdx.x;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(x + row * K);
    const int nchunk = K >> 3;
    u32x4 v[kNormChunks];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < kNormChunks; ++c) {
        const int at = t + c * kNormThreads;
        v[c] = at < nchunk ? src[at] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t word = v[c][e];
            const float lo = bf16_bits_to_float(word & 0xFFFFu), hi = bf16_bits_to_float(word >> 16);
            ss = fmaf(lo, lo, ss);
            ss = fmaf(hi, hi, ss);
        }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) ss += __shfl_xor(ss, m, 64);
    if ((t & 63) == 0) part[t >> 6] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < kNormThreads / 64; ++i) total += part[i];
    const float rms = sqrtf(total / (float)K + eps);
    u32x4 *dst = reinterpret_cast<u32x4 *>(out + row * K);
    const u32x4 *wsrc = reinterpret_cast<const u32x4 *>(w);
#pragma unroll
    for (int c = 0; c < kNormChunks; ++c) {
        const int at = t + c * kNormThreads;
        if (at < nchunk) {
            const u32x4 nw = wsrc[at];
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t word = v[c][e], wword = nw[e];
                const float lo = bf16_bits_to_float(word & 0xFFFFu), hi = bf16_bits_to_float(word >> 16);
                const float wl = bf16_bits_to_float(wword & 0xFFFFu), wh = bf16_bits_to_float(wword >> 16);
                o[e] = pack_bf16x2((lo / rms) * wl, (hi / rms) * wh);
            }
            dst[at] = o;
        }
    }
}

size_t round256(size_t n) { return (n + 255) / 256 * 256; }

}  // namespace

bool prefill_block_supported(int M, int E, int H) { return M > 0 && E > 0 && H > 0 && E % 8 == 0 && E <= 8 * kNormThreads * kNormChunks; }

constexpr int kPlanCus = 256;   // the split-K scratch is sized for this many CUs; a device with another count splits only if it fits

static size_t splitk_bytes(int M, int E, int H, int cus) {
    size_t b = gemm_prefill_splitk_bytes(M, E, E, cus);
    const size_t g = gemm_prefill_splitk_bytes(M, E, H, cus), d = gemm_prefill_splitk_bytes(M, H, E, cus);
    b = g > b ? g : b;
    return d > b ? d : b;
}

size_t prefill_block_scratch_bytes(int M, int E, int H) {
    return 2 * round256((size_t)M * E * sizeof(uint16_t)) + 2 * round256((size_t)M * H * sizeof(uint16_t)) +
           round256(splitk_bytes(M, E, H, kPlanCus));
}

hipError_t launch_rmsnorm_rows(const uint16_t *x, const uint16_t *w, uint16_t *out, int M, int K, float eps, hipStream_t stream) {
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(M), dim3(kNormThreads), 0, stream, x, w, out, K, eps);
    return hipGetLastError();
}

// The reference's 6-launch prefill ELF rms_gemms_rope_int4
// (programming_examples/llms/llama32_1b_int4/multi_launch_builder/rms_gemms_rope_int4_multi.py:4-17, CPU reference
// :414-436, 543-561) as two launches: row-wise RMSNorm, then one GEMM over the Q|K|V weights concatenated along
// N whose epilogue rotates the Q and K heads (row m at position pos0 + m).
hipError_t launch_prefill_rms_qkv_rope(const uint16_t *x, const uint16_t *norm_w, float eps, const PrefillLinear &wqkv,
                                       const uint16_t *rope_lut, int pos0, uint16_t *qkv_out, int M, int E, int n_heads,
                                       int n_kv, int head_dim, uint16_t *normed, hipStream_t stream) {
    hipError_t e = launch_rmsnorm_rows(x, norm_w, normed, M, E, eps, stream);
    if (e != hipSuccess) return e;
    const GemmRope rope = {(n_heads + n_kv) * head_dim, head_dim, pos0};
    return launch_gemm_prefill(normed, wqkv.qw, wqkv.qz, wqkv.sc, qkv_out, M, E, (n_heads + 2 * n_kv) * head_dim, stream,
                               kEpiRope, rope_lut, nullptr, 0, &rope);
}

hipError_t launch_prefill_o_ffn(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_w, float eps,
                                const PrefillLinear &wo, const PrefillLinear &wg, const PrefillLinear &wu,
                                const PrefillLinear &wd, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                int H, void *workspace, int cus, hipStream_t stream) {
    char *base = static_cast<char *>(workspace);
    uint16_t *res1 = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * E * sizeof(uint16_t));
    uint16_t *normed = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * E * sizeof(uint16_t));
    uint16_t *gate = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * H * sizeof(uint16_t));
    uint16_t *h = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * H * sizeof(uint16_t));
    // split-K partial products of the launches that have too few tiles for the chip
    float *sk = splitk_bytes(M, E, H, cus) <= splitk_bytes(M, E, H, kPlanCus) && splitk_bytes(M, E, H, cus) > 0
                    ? reinterpret_cast<float *>(base) : nullptr;
    if (res1_out) res1 = res1_out;
    if (h_out) h = h_out;
    hipError_t e = launch_gemm_prefill(attn_out, wo.qw, wo.qz, wo.sc, res1, M, E, E, stream, kEpiAddRounded, x_residual, sk, cus);
    if (e != hipSuccess) return e;
    e = launch_rmsnorm_rows(res1, ffn_norm_w, normed, M, E, eps, stream);
    if (e != hipSuccess) return e;
    e = launch_gemm_prefill(normed, wg.qw, wg.qz, wg.sc, gate, M, E, H, stream, kEpiNone, nullptr, sk, cus);
    if (e != hipSuccess) return e;
    e = launch_gemm_prefill(normed, wu.qw, wu.qz, wu.sc, h, M, E, H, stream, kEpiSiluGateMul, gate, sk, cus);
    if (e != hipSuccess) return e;
    return launch_gemm_prefill(h, wd.qw, wd.qz, wd.sc, y, M, H, E, stream, kEpiAddRounded, res1, sk, cus);
}

// The same two blocks on stream-order weights (gemm_ws.hip): no split-K scratch, the narrow-tile choice of that kernel
// covers the projections with few tiles.
bool prefill_block_stream_supported(int M, int E, int H) {
    return prefill_block_supported(M, E, H) && gemm_prefill_ws_supported(M, E, E) && gemm_prefill_ws_supported(M, E, H) &&
           gemm_prefill_ws_supported(M, H, E);
}

hipError_t launch_prefill_rms_qkv_rope_stream(const uint16_t *x, const uint16_t *norm_w, float eps, const void *wqkv,
                                              const uint16_t *rope_lut, int pos0, uint16_t *qkv_out, int M, int E, int n_heads,
                                              int n_kv, int head_dim, uint16_t *normed, hipStream_t stream, bool q4) {
    hipError_t e = launch_rmsnorm_rows(x, norm_w, normed, M, E, eps, stream);
    if (e != hipSuccess) return e;
    const GemmRope rope = {(n_heads + n_kv) * head_dim, head_dim, pos0};
    return launch_gemm_prefill_ws(normed, wqkv, qkv_out, M, E, (n_heads + 2 * n_kv) * head_dim, stream, kEpiRope, rope_lut, &rope, q4);
}

hipError_t launch_prefill_o_ffn_stream(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_w, float eps,
                                       const void *wo, const void *wg, const void *wu, const void *wd, uint16_t *y,
                                       uint16_t *res1_out, uint16_t *h_out, int M, int E, int H, void *workspace,
                                       hipStream_t stream, bool q4) {
    char *base = static_cast<char *>(workspace);
    uint16_t *res1 = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * E * sizeof(uint16_t));
    uint16_t *normed = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * E * sizeof(uint16_t));
    uint16_t *gate = reinterpret_cast<uint16_t *>(base);
    base += round256((size_t)M * H * sizeof(uint16_t));
    uint16_t *h = reinterpret_cast<uint16_t *>(base);
    if (res1_out) res1 = res1_out;
    if (h_out) h = h_out;
    hipError_t e = launch_gemm_prefill_ws(attn_out, wo, res1, M, E, E, stream, kEpiAddRounded, x_residual, nullptr, q4);
    if (e != hipSuccess) return e;
    e = launch_rmsnorm_rows(res1, ffn_norm_w, normed, M, E, eps, stream);
    if (e != hipSuccess) return e;
    if (g_gemv_ws_tune.prefill_swiglu_split) {
        e = launch_gemm_prefill_ws(normed, wg, gate, M, E, H, stream, kEpiNone, nullptr, nullptr, q4);
        if (e != hipSuccess) return e;
        e = launch_gemm_prefill_ws(normed, wu, h, M, E, H, stream, kEpiSiluGateMul, gate, nullptr, q4);
    } else {
        e = launch_gemm_prefill_ws_swiglu(normed, wg, wu, h, M, E, H, stream, q4);
    }
    if (e != hipSuccess) return e;
    return launch_gemm_prefill_ws(h, wd, y, M, H, E, stream, kEpiAddRounded, res1, nullptr, q4);
}

}  // namespace w4a16
