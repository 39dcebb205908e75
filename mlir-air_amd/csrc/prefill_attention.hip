// Causal grouped-query attention over the M tokens of a prefill, for gfx950: the `flash_attn` step between the
// two int4 prefill ELFs of the reference (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:302-326;
// its CPU form attention_reference, softmax(Q K^T / sqrt(d) + causal mask) V per head in fp32).
//
// Input is the [M, (n_heads + 2 n_kv) * HD] tensor of w4a16_prefill_rms_qkv_rope_bf16 (roped Q | roped K | V per
// row); output attn_out bf16 [M, n_heads * HD].
//
// A workgroup of four waves shares the K and V rows of one KV head: a wave owns 32 queries of one query head, and
// the four waves are HPW heads of the KV head's group times 4 / HPW query blocks (HPW = 4 for the 32 / 8 head models:
// the four heads of a group meet the same keys at the same time, so no wave idles at the diagonal).  Keys go by in
// blocks of 64 (heads of 64) or 32 (heads of 128) through LDS, double buffered, one barrier per block; the rows travel global -> registers during the
// block before and registers -> LDS at the head of the block.  The online softmax keeps one running maximum and sum
// per query.  Everything is computed transposed so that a lane owns one query (of each of its two 16-query blocks)
// throughout (MFMA 16x16x32 bf16):
//   S^T[key, q] = K . Q^T      A = K rows from LDS (16-byte reads), B = Q^T held in registers
//   O^T[d, q]  += V^T . P^T    A = V^T, B = P^T built from the lane's own S^T registers
// Each A operand read serves both query blocks.  The D layout gives a lane keys 4g..4g+3 of each 16-key block
// (g = lane / 16) while the B operand wants 8 consecutive k per lane; since a sum over keys does not care about their
// order, k slot 8g + j of the second product is DEFINED as key (j < 4 ? 4g + j : 16 + 4g + j - 4) of the 32 keys of a
// K-step, so no cross-lane movement of P is needed.  V stays row-major in LDS ([key][d], as it arrives): the V^T
// operand comes from the transposing LDS read (ds_read_b64_tr_b16: within 16 lanes, lane i receives element i % 4 of
// the 8-byte chunks addressed by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12), lane j of a group pointing at key
// 4g + j / 4, columns 4 (j % 4) .. + 3 of the 16-column block: lane i then holds column i of keys 4g .. 4g + 3.
// Scores go to the log2 domain inside the exponential's argument (one fma), P is rounded to bf16 for the second
// product, the sum of P is kept in fp32 before that rounding.  Only the blocks on the diagonal are masked.
// Workgroups are dispatched last query block first (the longest key ranges first).
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

struct PrefillAttnParams {
    const uint16_t *qkv;
    uint16_t *out;
    int M, ld;               // tokens, row stride of qkv in elements
    int n_heads, n_kv;
    float scale_log2;        // log2(e) / sqrt(HD)
};

constexpr float kMasked = -1.0e30f;
// keys per block: 64 for heads of 64, 32 for heads of 128 (the same MFMA work per block; 64 keys of 128 elements
// in flight through the registers do not fit beside the 128-wide output with two workgroups per CU)
template <int HD>
constexpr int attn_keys() {
    return HD == 64 ? 64 : 32;
}

typedef short shortx4 __attribute__((ext_vector_type(4)));

template <int HD>
constexpr size_t attn_lds_bytes() {
    return 2 * (size_t)attn_keys<HD>() * ((HD + 8) + (HD + 16)) * sizeof(uint16_t);
}

// max over the four lanes ql, ql + 16, ql + 32, ql + 48
__device__ __forceinline__ float max_over_lane_groups(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);   // rows (0, 1) and (2, 3) exchanged
    v = fmaxf(__builtin_bit_cast(float, (uint32_t)a[0]), __builtin_bit_cast(float, (uint32_t)a[1]));
    const uint32_t w = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);   // halves exchanged
    return fmaxf(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}

template <int HD, int HPW>
__global__ void __launch_bounds__(256, 2) prefill_attn_kernel(const PrefillAttnParams p) {
    constexpr int KB = attn_keys<HD>(), NKK = KB / 16, NT = KB / 32;   // 16-key blocks of S^T, K-steps of the second product
    constexpr int KP = HD + 8;     // K tile row pitch (elements): 144 / 272 B, conflict-free 16-byte reads over 16 rows
    constexpr int VP = HD + 16;    // V tile row pitch: 160 / 288 B = 32 B mod 256, conflict-free transposing reads
    constexpr int QS = 4 / HPW;    // 32-query blocks per workgroup
    constexpr int QW = 32 * QS;
    extern __shared__ __attribute__((aligned(16))) uint16_t attn_lds[];
    uint16_t *kt = attn_lds;                  // [2][KB * KP]
    uint16_t *vt = attn_lds + 2 * KB * KP;    // [2][KB * VP]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ql = lane & 15, g = lane >> 4;
    const int G = p.n_heads / p.n_kv, groups = G / HPW;
    const int kvh = blockIdx.y / groups;
    const int head = kvh * G + (blockIdx.y % groups) * HPW + wave % HPW;
    const int qb = ((int)gridDim.x - 1 - (int)blockIdx.x) * QW;      // the longest key ranges are dispatched first
    const int q0 = qb + 32 * (wave / HPW);
    const int k_off = p.n_heads * HD + kvh * HD, v_off = (p.n_heads + p.n_kv) * HD + kvh * HD;

    int qi[2];
    bf16x8 qf[2][HD / 32];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        qi[b] = q0 + 16 * b + ql;                                      // this lane's queries (may be >= M in the last block)
        const int qrow = qi[b] < p.M ? qi[b] : p.M - 1;                // load in range, never stored
#pragma unroll
        for (int ks = 0; ks < HD / 32; ++ks)
            qf[b][ks] = *reinterpret_cast<const bf16x8 *>(p.qkv + (size_t)qrow * p.ld + head * HD + 32 * ks + 8 * g);
    }

    floatx4 o[2][HD / 16];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int d = 0; d < HD / 16; ++d) o[b][d] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m[2] = {kMasked, kMasked}, l[2] = {0.f, 0.f};   // running maximum of the raw scores, sum of exponentials

    const int kend = qb + QW < p.M ? qb + QW : p.M;       // causal: no query of the workgroup sees a later key
    const int nit = (kend + KB - 1) / KB;
    // A thread moves chunks c = tid (+ 256 i) of 8 elements: key c / (HD / 8), elements 8 (c % (HD / 8)) ..
    constexpr int CPR = HD / 8, NCH = KB * CPR / 256;
    u32x4 kreg[NCH], vreg[NCH];
    auto fetch = [&](int it) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            const int key = c / CPR, e8 = c % CPR;
            const int gk = it * KB + key < p.M ? it * KB + key : p.M - 1;
            const uint16_t *row = p.qkv + (size_t)gk * p.ld;
            kreg[i] = *reinterpret_cast<const u32x4 *>(row + k_off + 8 * e8);
            vreg[i] = *reinterpret_cast<const u32x4 *>(row + v_off + 8 * e8);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            const int key = c / CPR, e8 = c % CPR;
            *reinterpret_cast<u32x4 *>(&kt[buf * KB * KP + key * KP + 8 * e8]) = kreg[i];
            *reinterpret_cast<u32x4 *>(&vt[buf * KB * VP + key * VP + 8 * e8]) = vreg[i];
        }
    };

    // per-lane element offsets into a tile: K rows for the first product, the transposing read of V for the second
    const int k_lane = ql * KP + 8 * g;
    const int v_lane = (4 * g + (ql >> 2)) * VP + 4 * (ql & 3);

    auto block = [&](int it, int buf, auto MASKED) {
        constexpr bool kMask = decltype(MASKED)::value;
        const uint16_t *ktile = kt + buf * KB * KP, *vtile = vt + buf * KB * VP;
        const int kb = it * KB;
        floatx4 s[NKK][2];
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            s[kk][0] = s[kk][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < HD / 32; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(&ktile[k_lane + 16 * kk * KP + 32 * ks]);
                s[kk][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[0][ks], s[kk][0], 0, 0, 0);
                s[kk][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[1][ks], s[kk][1], 0, 0, 0);
            }
        }
        // s[kk][b][r] is the raw score of key kb + 16 kk + 4 g + r against query qi[b]
        bf16x8 pb[2][NT];   // [query block][K-step of 32 keys]
        float alpha[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if constexpr (kMask) {
#pragma unroll
                for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (kb + 16 * kk + 4 * g + r > qi[b]) s[kk][b][r] = kMasked;
            }
            float bm = fmaxf(fmaxf(s[0][b][0], s[0][b][1]), fmaxf(s[0][b][2], s[0][b][3]));
#pragma unroll
            for (int kk = 1; kk < NKK; ++kk) bm = fmaxf(fmaxf(bm, fmaxf(s[kk][b][0], s[kk][b][1])), fmaxf(s[kk][b][2], s[kk][b][3]));
            bm = max_over_lane_groups(bm);
            const float m_new = fmaxf(m[b], bm);               // finite from the first block on: key 0 is visible to every query
            const float msc = m_new * p.scale_log2;
            // v_exp_f32 directly: arguments are <= 0, results that would be denormal may flush to zero, and a masked
            // score (-1e30 against a finite maximum) gives exactly 0
            alpha[b] = __builtin_amdgcn_exp2f(m[b] * p.scale_log2 - msc);
            float psum = 0.f;
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(s[kk][b][r], p.scale_log2, -msc));
                    s[kk][b][r] = e;
                    psum += e;
                }
            l[b] = l[b] * alpha[b] + psum;
            m[b] = m_new;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                u32x4 pw;
                pw[0] = pack_bf16x2(s[2 * t][b][0], s[2 * t][b][1]);
                pw[1] = pack_bf16x2(s[2 * t][b][2], s[2 * t][b][3]);
                pw[2] = pack_bf16x2(s[2 * t + 1][b][0], s[2 * t + 1][b][1]);
                pw[3] = pack_bf16x2(s[2 * t + 1][b][2], s[2 * t + 1][b][3]);
                pb[b][t] = __builtin_bit_cast(bf16x8, pw);
            }
        }
        // the running maxima settle after a few blocks: the rescaling is skipped when no lane of the wave needs it
        if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.0f || alpha[1] != 1.0f) != 0) {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int d = 0; d < HD / 16; ++d) o[b][d] *= alpha[b];
        }
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int d = 0; d < HD / 16; ++d) {
                const uint16_t *src = &vtile[v_lane + 32 * t * VP + 16 * d];
                const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *)src);
                const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *)(src + 16 * VP));
                const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
                const u32x4 aw = {lo2.x, lo2.y, hi2.x, hi2.y};
                const bf16x8 a = __builtin_bit_cast(bf16x8, aw);
                o[0][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[0][t], o[0][d], 0, 0, 0);
                o[1][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[1][t], o[1][d], 0, 0, 0);
            }
    };

    fetch(0);
    stage(0);
    if (nit > 1) fetch(1);
    __syncthreads();
    for (int it = 0; it < nit; ++it) {
        const int buf = it & 1;
        if (it + 1 < nit) {
            stage(buf ^ 1);                      // read last during block it - 1, before the barrier that ended it
            if (it + 2 < nit) fetch(it + 2);
        }
        const int kb = it * KB;
        if (kb <= q0 + 31) {                     // else every key of the block is after this wave's queries
            if (kb + KB - 1 > q0) block(it, buf, std::true_type{});
            else block(it, buf, std::false_type{});
        }
        __syncthreads();
    }

#pragma unroll
    for (int b = 0; b < 2; ++b) {
        // the four lane groups of a query hold the sums over their own keys
        float lb = l[b];
        lb += __shfl_xor(lb, 16, 64);
        lb += __shfl_xor(lb, 32, 64);
        if (qi[b] >= p.M) continue;
        const float inv = 1.0f / lb;
        uint16_t *dst = p.out + (size_t)qi[b] * p.n_heads * HD + head * HD + 4 * g;
#pragma unroll
        for (int d = 0; d < HD / 16; ++d) {
            // o[b][d][r] is output element 16 d + 4 g + r of query qi[b]
            const uint2 w = uint2{pack_bf16x2(o[b][d][0] * inv, o[b][d][1] * inv), pack_bf16x2(o[b][d][2] * inv, o[b][d][3] * inv)};
            *reinterpret_cast<uint2 *>(dst + 16 * d) = w;
        }
    }
}

template <int HD, int HPW>
hipError_t launch_attn(const PrefillAttnParams &p, hipStream_t stream) {
    constexpr size_t lds = attn_lds_bytes<HD>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_attn_kernel<HD, HPW>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    constexpr int QW = 32 * (4 / HPW);
    const dim3 grid((p.M + QW - 1) / QW, p.n_kv * (p.n_heads / p.n_kv / HPW));
    hipLaunchKernelGGL((prefill_attn_kernel<HD, HPW>), grid, dim3(256), lds, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_prefill_attention(const uint16_t *qkv, uint16_t *attn_out, int M, int n_heads, int n_kv, int head_dim,
                                    hipStream_t stream) {
    PrefillAttnParams p;
    p.qkv = qkv;
    p.out = attn_out;
    p.M = M;
    p.ld = (n_heads + 2 * n_kv) * head_dim;
    p.n_heads = n_heads;
    p.n_kv = n_kv;
    p.scale_log2 = 1.4426950408889634f / sqrtf((float)head_dim);
    const int G = n_heads / n_kv;
    const int hpw = G % 4 == 0 ? 4 : G % 2 == 0 ? 2 : 1;   // query heads of one KV head per workgroup
    if (head_dim == 64)
        return hpw == 4 ? launch_attn<64, 4>(p, stream) : hpw == 2 ? launch_attn<64, 2>(p, stream) : launch_attn<64, 1>(p, stream);
    return hpw == 4 ? launch_attn<128, 4>(p, stream) : hpw == 2 ? launch_attn<128, 2>(p, stream) : launch_attn<128, 1>(p, stream);
}

}  // namespace w4a16
