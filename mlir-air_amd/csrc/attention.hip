// Single-query (decode) GQA attention over a bf16 KV cache, with the half-split RoPE of the new
// token's Q and K and the cache append fused in.
//
// Input is the fresh, un-rotated projection vector qkv = [Q (n_heads * HD) | K (n_kv * HD) |
// V (n_kv * HD)] of the current token.  HBM-bound on the cache: every cached K and V element is
// read once, by the one workgroup that owns its (kv head, sequence chunk), and used for all G
// query heads of the group.
//
//   grid  = (nsplit sequence chunks, n_kv heads), 4 waves per workgroup
//   lanes = HD / 8 lanes share one cache position (16-byte loads), so a wave covers 64 / (HD / 8)
//           positions per load; each lane group keeps a private online-softmax state
//           (m, l, acc[8]) per query head and the states are merged at the end: across lane
//           groups with shuffles, across waves through LDS, across chunks by the combine kernel
//   the chunk that holds `pos` first rotates K, stores K and V of the new token into the caches,
//   and then reads them back like any other position
//
// Rounding points follow the reference's decode step: Q and K are rounded to bf16 after RoPE,
// scores, softmax and the weighted sum are fp32, the output is rounded to bf16 once.
#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

constexpr float kNegBig = kAttnNegBig;
constexpr float kLog2e = 1.4426950408889634f;

struct AttnParams {
    const uint16_t *qkv;
    const uint16_t *lut;      // [HD]: cos[0..HD/2), sin[0..HD/2) at position pos
    uint16_t *k_cache;        // [n_kv, max_seq, HD]
    uint16_t *v_cache;
    uint16_t *out;            // [n_heads * HD]
    float *part_ml;           // [n_heads, nsplit, 2]
    float *part_acc;          // [n_heads, nsplit, HD]
    int pos, max_seq, n_heads, n_kv, nsplit, chunk;
    float scale;
};

__device__ __forceinline__ void unpack8(const u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = __builtin_bit_cast(float, v[j] << 16);
        f[2 * j + 1] = __builtin_bit_cast(float, v[j] & 0xFFFF0000u);
    }
}

// 2^x for x <= 0 as the bare v_exp_f32: the library routine's rescaling of very negative arguments only
// changes results below 2^-126, which vanish against the running sums they are added to.
__device__ __forceinline__ float exp2_nonpos(float x) { return __builtin_amdgcn_exp2f(x); }

// Sum over a group of LPP = 8 or 16 neighbouring lanes (a group never crosses a row of 16 lanes), every lane
// of the group receiving the sum: an xor butterfly on data-parallel-primitive moves (quad permutes for
// distances 1 and 2, half-row and row mirrors for 4 and 8: once the quads agree, mirroring meets the
// partner quad), i.e. full-rate VALU adds instead of LDS-routed shuffles.  Bit-identical to the butterfly
// with shuffles: every step adds the same two partial sums.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return v + __builtin_bit_cast(float, moved);
}
template <int LPP>
__device__ __forceinline__ float group_sum(float s) {
    static_assert(LPP == 8 || LPP == 16, "lane groups of 8 or 16");
    s = dpp_add<0xB1>(s);    // quad_perm [1, 0, 3, 2]
    s = dpp_add<0x4E>(s);    // quad_perm [2, 3, 0, 1]
    s = dpp_add<0x141>(s);   // row_half_mirror
    if constexpr (LPP == 16) s = dpp_add<0x140>(s);   // row_mirror
    return s;
}

// Half-split RoPE of elements [e0, e0 + 8) of one head: x at src, rounded to bf16 (returned as floats).
template <int HD>
__device__ __forceinline__ void rope8(const uint16_t *src, const uint16_t *lut, int e0, float (&out)[8]) {
    constexpr int HALF = HD / 2;
    const bool low = e0 < HALF;
    const int i0 = low ? e0 : e0 - HALF;
    float x[8], y[8], c[8], s[8];
    unpack8(*reinterpret_cast<const u32x4 *>(src + e0), x);
    unpack8(*reinterpret_cast<const u32x4 *>(src + (low ? e0 + HALF : e0 - HALF)), y);
    unpack8(*reinterpret_cast<const u32x4 *>(lut + i0), c);
    unpack8(*reinterpret_cast<const u32x4 *>(lut + HALF + i0), s);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        // low half: x1 cos - x2 sin; high half: x2 cos + x1 sin (x is the lane's own element)
        const float r = low ? x[j] * c[j] - y[j] * s[j] : x[j] * c[j] + y[j] * s[j];
        out[j] = bf16_bits_to_float(float_to_bf16_bits(r));
    }
}

template <int HD, int G>
__global__ void __launch_bounds__(256) attn_partial_kernel(const AttnParams p) {
    constexpr int LPP = HD / 8;        // lanes per position
    constexpr int PPW = 64 / LPP;      // positions per wave and load
    constexpr int STATE = 2 + HD;      // m, l, acc[HD] per head
    __shared__ float sh[4 * G * STATE];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPP, slot = lane / LPP;
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int seq_len = p.pos + 1;
    const int t0 = split * p.chunk;
    const int t1 = min(seq_len, t0 + p.chunk);
    const int nq = p.n_heads * HD, nkv = p.n_kv * HD;

    uint16_t *kc = p.k_cache + (size_t)kvh * p.max_seq * HD;
    uint16_t *vc = p.v_cache + (size_t)kvh * p.max_seq * HD;

    // the chunk that owns `pos` appends the new token's K (rotated) and V
    if (t0 <= p.pos && p.pos < t1) {
        if (threadIdx.x < LPP) {
            float kr[8];
            rope8<HD>(p.qkv + nq + kvh * HD, p.lut, 8 * sub, kr);
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = pack_bf16x2(kr[2 * j], kr[2 * j + 1]);
            *reinterpret_cast<u32x4 *>(kc + (size_t)p.pos * HD + 8 * sub) = o;
            *reinterpret_cast<u32x4 *>(vc + (size_t)p.pos * HD + 8 * sub) =
                *reinterpret_cast<const u32x4 *>(p.qkv + nq + nkv + kvh * HD + 8 * sub);
        }
        __syncthreads();
    }

    // rotated, bf16-rounded query slices of the G heads, pre-scaled for exp2
    float q[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        rope8<HD>(p.qkv + (size_t)(kvh * G + h) * HD, p.lut, 8 * sub, q[h]);
#pragma unroll
        for (int j = 0; j < 8; ++j) q[h][j] *= p.scale * kLog2e;
    }

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        m[h] = kNegBig;
        l[h] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[h][j] = 0.f;
    }

    // UN positions per lane are requested together, so that a chunk costs one or two memory
    // round trips instead of one per position
    constexpr int UN = G == 8 ? 2 : 4;
    for (int tb = t0 + wave * PPW + slot; tb < t1; tb += UN * 4 * PPW) {
        u32x4 kraw[UN], vraw[UN];
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const int t = tb + i * 4 * PPW;
            const int tc = t < t1 ? t : t0;   // in range; the result of a clamped slot is discarded
            kraw[i] = *reinterpret_cast<const u32x4 *>(kc + (size_t)tc * HD + 8 * sub);
            vraw[i] = *reinterpret_cast<const u32x4 *>(vc + (size_t)tc * HD + 8 * sub);
        }
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            if (tb + i * 4 * PPW >= t1) break;   // uniform within a lane group
            float k[8], v[8];
            unpack8(kraw[i], k);
            unpack8(vraw[i], v);
#pragma unroll
            for (int h = 0; h < G; ++h) {
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) s = fmaf(q[h][j], k[j], s);
                s = group_sum<LPP>(s);
                const float mn = fmaxf(m[h], s);
                const float corr = exp2_nonpos(m[h] - mn);
                const float pr = exp2_nonpos(s - mn);
                m[h] = mn;
                l[h] = l[h] * corr + pr;
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[h][j] = fmaf(pr, v[j], acc[h][j] * corr);
            }
        }
    }

    // merge the lane groups of the wave (lanes with equal `sub`)
#pragma unroll
    for (int off = LPP; off < 64; off <<= 1) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            const float m2 = __shfl_xor(m[h], off), l2 = __shfl_xor(l[h], off);
            const float mn = fmaxf(m[h], m2);
            const float c1 = exp2_nonpos(m[h] - mn), c2 = exp2_nonpos(m2 - mn);
            m[h] = mn;
            l[h] = l[h] * c1 + l2 * c2;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[h][j] = acc[h][j] * c1 + __shfl_xor(acc[h][j], off) * c2;
        }
    }
    if (slot == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float *dst = sh + (wave * G + h) * STATE;
            if (sub == 0) {
                dst[0] = m[h];
                dst[1] = l[h];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[2 + 8 * sub + j] = acc[h][j];
        }
    }
    __syncthreads();

    // merge the four waves; one thread per (head, element)
    for (int idx = threadIdx.x; idx < G * HD; idx += 256) {
        const int h = idx / HD, e = idx % HD;
        float mn = kNegBig;
#pragma unroll
        for (int w = 0; w < 4; ++w) mn = fmaxf(mn, sh[(w * G + h) * STATE]);
        float ls = 0.f, as = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float *src = sh + (w * G + h) * STATE;
            const float c = exp2f(src[0] - mn);
            ls += src[1] * c;
            as += src[2 + e] * c;
        }
        const int head = kvh * G + h;
        if (p.nsplit == 1) {
            p.out[(size_t)head * HD + e] = float_to_bf16_bits(as / ls);
        } else {
            const size_t slot_idx = (size_t)head * p.nsplit + split;
            if (e == 0) {
                p.part_ml[2 * slot_idx] = mn;
                p.part_ml[2 * slot_idx + 1] = ls;
            }
            p.part_acc[slot_idx * HD + e] = as;
        }
    }
}

// out[head] = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M); grid = n_heads, block = HD threads.
// The chunk weights are computed once by the first wave (lane s owns chunk s, nsplit <= 32).
__global__ void attn_combine_kernel(const float *part_ml, const float *part_acc, uint16_t *out, int nsplit, int hd) {
    __shared__ float wgt[kMaxAttnSplit];
    __shared__ float inv_l;
    const int head = blockIdx.x, e = threadIdx.x;
    // every load of the kernel is requested up front: one memory round trip in total
    const float *src = part_acc + (size_t)head * nsplit * hd + e;
    float a[kMaxAttnSplit];
#pragma unroll
    for (int s = 0; s < kMaxAttnSplit; ++s) a[s] = s < nsplit ? src[(size_t)s * hd] : 0.f;
    if (e < 64) {
        const bool live = e < nsplit;
        const float m = live ? part_ml[2 * ((size_t)head * nsplit + e)] : kNegBig;
        const float l = live ? part_ml[2 * ((size_t)head * nsplit + e) + 1] : 0.f;
        const float mn = wave_reduce<true>(m);
        const float c = exp2f(m - mn);
        const float ls = wave_reduce<false>(l * c);
        if (e < kMaxAttnSplit) wgt[e] = live ? c : 0.f;
        if (e == 0) inv_l = 1.0f / ls;
    }
    __syncthreads();
    float as = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxAttnSplit; ++s) as = fmaf(a[s], wgt[s], as);
    out[(size_t)head * hd + e] = float_to_bf16_bits(as * inv_l);
}

template <int HD>
hipError_t launch_g(int g, const AttnParams &p, dim3 grid, hipStream_t stream) {
    switch (g) {
        case 1: hipLaunchKernelGGL((attn_partial_kernel<HD, 1>), grid, dim3(256), 0, stream, p); break;
        case 2: hipLaunchKernelGGL((attn_partial_kernel<HD, 2>), grid, dim3(256), 0, stream, p); break;
        case 4: hipLaunchKernelGGL((attn_partial_kernel<HD, 4>), grid, dim3(256), 0, stream, p); break;
        case 8: hipLaunchKernelGGL((attn_partial_kernel<HD, 8>), grid, dim3(256), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

int attention_nsplit(int seq_len) {
    int n = (seq_len + 63) / 64;   // >= 64 positions per chunk
    if (n > kMaxAttnSplit) n = kMaxAttnSplit;
    return n < 1 ? 1 : n;
}

size_t attention_workspace_bytes(int n_heads, int head_dim) {
    return (size_t)n_heads * kMaxAttnSplit * (2 + (size_t)head_dim) * sizeof(float);
}

hipError_t launch_decode_attention(const uint16_t *qkv, const uint16_t *lut_row, uint16_t *k_cache, uint16_t *v_cache,
                                   uint16_t *out, int pos, int max_seq, int n_heads, int n_kv, int head_dim,
                                   void *workspace, hipStream_t stream, bool combine) {
    AttnParams p;
    p.qkv = qkv;
    p.lut = lut_row;
    p.k_cache = k_cache;
    p.v_cache = v_cache;
    p.out = out;
    p.pos = pos;
    p.max_seq = max_seq;
    p.n_heads = n_heads;
    p.n_kv = n_kv;
    p.nsplit = attention_nsplit(pos + 1);
    const int ppb = 4 * (64 / (head_dim / 8));   // positions per workgroup iteration
    p.chunk = (((pos + 1 + p.nsplit - 1) / p.nsplit + ppb - 1) / ppb) * ppb;
    p.scale = 1.0f / sqrtf((float)head_dim);
    p.part_ml = reinterpret_cast<float *>(workspace);
    p.part_acc = p.part_ml + (size_t)n_heads * kMaxAttnSplit * 2;
    const dim3 grid(p.nsplit, n_kv);
    hipError_t e = head_dim == 64 ? launch_g<64>(n_heads / n_kv, p, grid, stream)
                                  : launch_g<128>(n_heads / n_kv, p, grid, stream);
    if (e != hipSuccess || p.nsplit == 1 || !combine) return e;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(n_heads), dim3(head_dim), 0, stream, p.part_ml, p.part_acc, out,
                       p.nsplit, head_dim);
    return hipGetLastError();
}

// Half-split RoPE of `rows` independent rows of `dim` elements, each with its own LUT row
// (cos then sin).  One thread rotates 8 consecutive elements of one row; dim % 16 == 0.
__global__ void __launch_bounds__(256) rope_rows_kernel(const uint16_t *x, const uint16_t *lut, uint16_t *out, int rows,
                                                        int dim) {
    const int per_row = dim >> 3;
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= rows * per_row) return;
    const int row = t / per_row, e0 = 8 * (t % per_row);
    const int half = dim >> 1;
    const bool low = e0 < half;
    const int i0 = low ? e0 : e0 - half;
    const uint16_t *src = x + (size_t)row * dim;
    const uint16_t *l = lut + (size_t)row * dim;
    float a[8], b[8], c[8], s[8];
    unpack8(*reinterpret_cast<const u32x4 *>(src + e0), a);
    unpack8(*reinterpret_cast<const u32x4 *>(src + (low ? e0 + half : e0 - half)), b);
    unpack8(*reinterpret_cast<const u32x4 *>(l + i0), c);
    unpack8(*reinterpret_cast<const u32x4 *>(l + half + i0), s);
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // products of two bf16 values are exact in fp32: one rounding to fp32, one to bf16, as in NumPy
        const float r0 = low ? a[2 * j] * c[2 * j] - b[2 * j] * s[2 * j] : a[2 * j] * c[2 * j] + b[2 * j] * s[2 * j];
        const float r1 = low ? a[2 * j + 1] * c[2 * j + 1] - b[2 * j + 1] * s[2 * j + 1]
                             : a[2 * j + 1] * c[2 * j + 1] + b[2 * j + 1] * s[2 * j + 1];
        o[j] = pack_bf16x2(r0, r1);
    }
    *reinterpret_cast<u32x4 *>(out + (size_t)row * dim + e0) = o;
}

hipError_t launch_rope_rows(const uint16_t *x, const uint16_t *lut, uint16_t *out, int rows, int dim, hipStream_t stream) {
    const int threads = rows * (dim >> 3);
    hipLaunchKernelGGL(rope_rows_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, x, lut, out, rows, dim);
    return hipGetLastError();
}

}  // namespace w4a16
