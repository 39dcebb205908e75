// Causal grouped-query attention over the M tokens of a prefill, for gfx950: the `flash_attn` step between the
// two int4 prefill ELFs of the reference (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:302-326;
// its CPU form attention_reference, softmax(Q K^T / sqrt(d) + causal mask) V per head in fp32).
//
// Input is the [M, (n_heads + 2 n_kv) * HD] tensor of w4a16_prefill_rms_qkv_rope_bf16 (roped Q | roped K | V per
// row); output attn_out bf16 [M, n_heads * HD].  One workgroup = 64 queries of one head, one wave = 16 of them.
// Keys go by in blocks of 32 through LDS; the online softmax keeps one running maximum and sum per query.
// Everything is computed transposed so that a lane owns one query throughout (MFMA 16x16x32 bf16):
//   S^T[key, q] = K . Q^T      A = K rows from LDS (16-byte reads), B = Q^T held in registers
//   O^T[d, q]  += V^T . P^T    A = V^T from LDS, B = P^T built from the lane's own S^T registers
// The D layout gives a lane keys 4g..4g+3 of each 16-key half (g = lane / 16) while the B operand wants 8
// consecutive k per lane; since a sum over keys does not care about their order, k slot 8g + j of the second
// product is DEFINED as key (j < 4 ? 4g + j : 16 + 4g + j - 4), and the V^T tile is written to LDS with its key
// columns in that order.  No cross-lane movement of P is needed.
// Scores are scaled into the log2 domain (exp2), P is rounded to bf16 for the second product, the sum of P
// is kept in fp32 before that rounding.
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

template <int HD>
__global__ void __launch_bounds__(256) prefill_attn_kernel(const PrefillAttnParams p) {
    constexpr int KP = HD + 8;     // K tile row pitch (elements): 144 / 272 B, conflict-free 16-byte reads over 16 rows
    constexpr int VP = 32 + 8;     // V^T tile row pitch: 80 B
    __shared__ __attribute__((aligned(16))) uint16_t kt[32 * KP];
    __shared__ __attribute__((aligned(16))) uint16_t vt[HD * VP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ql = lane & 15, g = lane >> 4;
    const int head = blockIdx.y, kvh = head / (p.n_heads / p.n_kv);
    const int qb = blockIdx.x * 64;
    const int q0 = qb + 16 * wave;
    const int qi = q0 + ql;                                   // this lane's query (may be >= M in the last block)
    const int qrow = qi < p.M ? qi : p.M - 1;                 // load in range, never stored
    const int k_off = p.n_heads * HD + kvh * HD, v_off = (p.n_heads + p.n_kv) * HD + kvh * HD;

    bf16x8 qf[HD / 32];
#pragma unroll
    for (int ks = 0; ks < HD / 32; ++ks)
        qf[ks] = *reinterpret_cast<const bf16x8 *>(p.qkv + (size_t)qrow * p.ld + head * HD + 32 * ks + 8 * g);

    floatx4 o[HD / 16];
#pragma unroll
    for (int d = 0; d < HD / 16; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m = kMasked, l = 0.f;

    const int kend = qb + 64 < p.M ? qb + 64 : p.M;           // causal: no query of the workgroup sees a later key
    // K and V rows of the next block travel global -> registers while the current block is multiplied, then
    // registers -> LDS between the two barriers.  A thread moves chunk c = tid (+ 256) of 8 elements: key c % 32, elements 8 (c / 32)..
    constexpr int NCH = 32 * HD / 8 / 256;
    u32x4 kreg[NCH], vreg[NCH];
    auto fetch = [&](int kb) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            const int key = c & 31, e8 = c >> 5;
            const int gk = kb + key < p.M ? kb + key : p.M - 1;
            const uint16_t *row = p.qkv + (size_t)gk * p.ld;
            kreg[i] = *reinterpret_cast<const u32x4 *>(row + k_off + 8 * e8);
            vreg[i] = *reinterpret_cast<const u32x4 *>(row + v_off + 8 * e8);
        }
    };
    fetch(0);
    for (int kb = 0; kb < kend; kb += 32) {
        __syncthreads();                                       // the previous block's tiles have been read
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid + 256 * i;
            const int key = c & 31, e8 = c >> 5;                // lanes = keys: the 2-byte V^T stores of a half-wave fill 64 contiguous bytes of one row
            *reinterpret_cast<u32x4 *>(&kt[key * KP + 8 * e8]) = kreg[i];
            // key -> k slot of the second product: half b = key / 16, r = key % 16: slot 8 (r / 4) + r % 4 + 4 b
            const int slot = 8 * ((key & 15) >> 2) + (key & 3) + 4 * (key >> 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t word = vreg[i][e];
                vt[(8 * e8 + 2 * e) * VP + slot] = (uint16_t)(word & 0xFFFFu);
                vt[(8 * e8 + 2 * e + 1) * VP + slot] = (uint16_t)(word >> 16);
            }
        }
        __syncthreads();
        if (kb + 32 < kend) fetch(kb + 32);
        if (kb > q0 + 15) continue;                            // every key of the block is after this wave's queries

        floatx4 s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            s[b] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < HD / 32; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(&kt[(16 * b + ql) * KP + 32 * ks + 8 * g]);
                s[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[ks], s[b], 0, 0, 0);
            }
        }
        // s[b][r] is the score of key kb + 16 b + 4 g + r against query qi
        float bm = kMasked;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = kb + 16 * b + 4 * g + r;
                const float v = (key > qi || key >= p.M) ? kMasked : s[b][r] * p.scale_log2;
                s[b][r] = v;
                bm = fmaxf(bm, v);
            }
        bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);                      // finite from the first block on: key 0 is visible to every query
        // v_exp_f32 directly: arguments are <= 0, results that would be denormal may flush to zero, and a masked
        // score (-1e30 minus a finite maximum) gives exactly 0
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);
        float psum = 0.f;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(s[b][r] - m_new);
                s[b][r] = e;
                psum += e;
            }
        l = l * alpha + psum;
        m = m_new;
        u32x4 pw;
        pw[0] = pack_bf16x2(s[0][0], s[0][1]);
        pw[1] = pack_bf16x2(s[0][2], s[0][3]);
        pw[2] = pack_bf16x2(s[1][0], s[1][1]);
        pw[3] = pack_bf16x2(s[1][2], s[1][3]);
        const bf16x8 pb = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
        for (int d = 0; d < HD / 16; ++d) {
            o[d] *= alpha;
            const bf16x8 a = *reinterpret_cast<const bf16x8 *>(&vt[(16 * d + ql) * VP + 8 * g]);
            o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, o[d], 0, 0, 0);
        }
    }
    // the four lane groups of a query hold the sums over their own keys
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (qi >= p.M) return;
    const float inv = 1.0f / l;
    uint16_t *dst = p.out + (size_t)qi * p.n_heads * HD + head * HD + 4 * g;
#pragma unroll
    for (int d = 0; d < HD / 16; ++d) {
        // o[d][r] is output element 16 d + 4 g + r of query qi
        const uint2 w = uint2{pack_bf16x2(o[d][0] * inv, o[d][1] * inv), pack_bf16x2(o[d][2] * inv, o[d][3] * inv)};
        *reinterpret_cast<uint2 *>(dst + 16 * d) = w;
    }
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
    const dim3 grid((M + 63) / 64, n_heads);
    if (head_dim == 64)
        hipLaunchKernelGGL(prefill_attn_kernel<64>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(prefill_attn_kernel<128>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

}  // namespace w4a16
