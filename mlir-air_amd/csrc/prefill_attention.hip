// Causal grouped-query attention over the M tokens of a prefill, for gfx950: the `flash_attn` step between the
// two int4 prefill ELFs of the reference (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:302-326;
// its CPU form attention_reference, softmax(Q K^T / sqrt(d) + causal mask) V per head in fp32).
//
// Input is the [M, (n_heads + 2 n_kv) * HD] tensor of w4a16_prefill_rms_qkv_rope_bf16 (roped Q | roped K | V per
// row); output attn_out bf16 [M, n_heads * HD].
//
// A workgroup is two sets of four waves on one KV head.  A wave owns 32 queries of one query head; the four waves of a
// set are HPW heads of the KV head's group times 4 / HPW query blocks (HPW = 4 for the 32 / 8 head models: the four
// heads of a group meet the same keys at the same time, so no wave idles at the diagonal) and share the K and V rows
// that go through LDS: an "item" of 32 * 4 / HPW queries.  Causal items differ in length by the number of items, so
// the workgroup takes a pair, the j-th longest with the j-th shortest (nA + nB key blocks, the same for every pair):
// set 0 runs the first half of that many blocks of the long item, set 1 the short item and then the long item's
// remaining blocks, and the two partial results of the long item are merged through LDS at the end.  Every wave of
// the chip then has the same number of blocks to do, whichever CU its workgroup lands on.  Keys go by in
// blocks of 64 through LDS, double buffered, one barrier per block; the rows travel global -> registers during the
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
// product, and the sum of P is a third product, a row of ones times P^T (the normaliser is the sum of the very
// weights that multiply V; the additions leave the VALU, which bounds this kernel).  Only the blocks on the diagonal
// are masked.

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
constexpr float kLazy = 8.0f;   // the reference maximum of the softmax may lag the true one by this much (log2 domain)
constexpr int kAttnKeys = 64;   // keys per block (heads of 128: 54 us at 64 keys, 60 us at 32, M = 2048, 32 / 8 heads)

typedef short shortx4 __attribute__((ext_vector_type(4)));

// two wave sets x two buffers of a K tile and a V tile; the exchange of partial results at the end reuses the space
template <int HD>
constexpr size_t attn_lds_bytes() {
    constexpr size_t tiles = 2 * 2 * (size_t)kAttnKeys * ((HD + 8) + (HD + 16)) * sizeof(uint16_t);
    constexpr size_t exchange = 4 * (2 * (HD / 16) * 4 + 4) * 64 * sizeof(float);
    return tiles > exchange ? tiles : exchange;
}

// (This file is compiled with -fno-honor-nans: otherwise every MFMA result is canonicalised before it enters a
// maximum, one more instruction per score.  A NaN in the inputs gives unspecified output values.)
__device__ __forceinline__ float max2(float a, float b) { return fmaxf(a, b); }

// max over the four lanes ql, ql + 16, ql + 32, ql + 48
__device__ __forceinline__ float max_over_lane_groups(float v) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);   // rows (0, 1) and (2, 3) exchanged
    v = max2(__builtin_bit_cast(float, (uint32_t)a[0]), __builtin_bit_cast(float, (uint32_t)a[1]));
    const uint32_t w = __builtin_bit_cast(uint32_t, v);
    const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);   // halves exchanged
    return max2(__builtin_bit_cast(float, (uint32_t)b[0]), __builtin_bit_cast(float, (uint32_t)b[1]));
}

template <int HD, int HPW>
__global__ void __launch_bounds__(512) prefill_attn_kernel(const PrefillAttnParams p) {
    constexpr int KB = kAttnKeys, NKK = KB / 16, NT = KB / 32;   // 16-key blocks of S^T, K-steps of the second product
    constexpr int KP = HD + 8;     // K tile row pitch (elements): 144 / 272 B, conflict-free 16-byte reads over 16 rows
    constexpr int VP = HD + 16;    // V tile row pitch: 160 / 288 B = 32 B mod 256, conflict-free transposing reads
    constexpr int QS = 4 / HPW;    // 32-query blocks per wave set
    constexpr int QW = 32 * QS;    // queries of an item
    constexpr int kTile = KB * (KP + VP);   // elements of one K + V tile
    extern __shared__ __attribute__((aligned(16))) uint16_t attn_lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int set = wave >> 2, w4 = wave & 3, tid4 = tid & 255;   // wave set 0 / 1, wave and thread within the set
    const int ql = lane & 15, g = lane >> 4;
    const int G = p.n_heads / p.n_kv, groups = G / HPW;
    const int kvh = blockIdx.y / groups;
    const int head = kvh * G + (blockIdx.y % groups) * HPW + w4 % HPW;
    const int k_off = p.n_heads * HD + kvh * HD, v_off = (p.n_heads + p.n_kv) * HD + kvh * HD;
    uint16_t *kt = attn_lds + set * 2 * kTile;   // this set's tiles: [2][K tile | V tile]

    // The workgroup's two items: the heavy one (many keys) and its light partner, nA + nB key blocks in all.  Set 0
    // takes the first hA = ceil((nA + nB) / 2) blocks of the heavy item; set 1 takes the light item and then the rest
    // of the heavy item's blocks (those at the diagonal), whose partial result set 0 merges into its own at the end.
    const int nx = (p.M + QW - 1) / QW;
    const int xa = nx - 1 - (int)blockIdx.x, xb = (int)blockIdx.x;
    auto blocks_of = [&](int x) {
        const int kend = (x + 1) * QW < p.M ? (x + 1) * QW : p.M;   // causal: no query of the item sees a later key
        return (kend + KB - 1) / KB;
    };
    const int nA = blocks_of(xa), nB = xb < xa ? blocks_of(xb) : 0;
    const int hA = (nA + nB + 1) / 2;
    // key block of this set's step s (or -1: nothing to do)
    auto block_of_step = [&](int s) {
        if (set == 0) return s < hA ? s : -1;
        if (s < nB) return s;
        const int it = hA + (s - nB);
        return it < nA ? it : -1;
    };

    int q0, qi[2];
    bf16x8 qf[2][HD / 32];
    floatx4 o[2][HD / 16];
    float m[2];         // reference maximum of the raw scores (may lag the true maximum by kLazy in the log2 domain)
    floatx4 l[2];       // sum of the bf16 probabilities: the product of a row of ones with P^T, every register the same
    auto begin_item = [&](int x) {
        q0 = x * QW + 32 * (w4 / HPW);
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            qi[b] = q0 + 16 * b + ql;                                      // this lane's queries (may be >= M in the last item)
            const int qrow = qi[b] < p.M ? qi[b] : p.M - 1;                // load in range, never stored
#pragma unroll
            for (int ks = 0; ks < HD / 32; ++ks)
                qf[b][ks] = *reinterpret_cast<const bf16x8 *>(p.qkv + (size_t)qrow * p.ld + head * HD + 32 * ks + 8 * g);
#pragma unroll
            for (int d = 0; d < HD / 16; ++d) o[b][d] = floatx4{0.f, 0.f, 0.f, 0.f};
            m[b] = kMasked;
            l[b] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        // the queries have arrived before the first block is requested: with these loads possibly in flight the
        // compiler waits for everything requested since, block in flight included, before the first MFMA of each step
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    };
    auto store_item = [&]() {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if (qi[b] >= p.M) continue;
            const float inv = 1.0f / l[b][0];
            uint16_t *dst = p.out + (size_t)qi[b] * p.n_heads * HD + head * HD + 4 * g;
#pragma unroll
            for (int d = 0; d < HD / 16; ++d) {
                // o[b][d][r] is output element 16 d + 4 g + r of query qi[b]
                const uint2 w = uint2{pack_bf16x2(o[b][d][0] * inv, o[b][d][1] * inv), pack_bf16x2(o[b][d][2] * inv, o[b][d][3] * inv)};
                *reinterpret_cast<uint2 *>(dst + 16 * d) = w;
            }
        }
    };

    // A thread of the set moves chunks c = tid4 (+ 256 i) of 8 elements: key c / (HD / 8), elements 8 (c % (HD / 8)) ..
    constexpr int CPR = HD / 8, NCH = KB * CPR / 256;
    u32x4 kreg[NCH], vreg[NCH];
    auto fetch = [&](int it) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = tid4 + 256 * i;
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
            const int c = tid4 + 256 * i;
            const int key = c / CPR, e8 = c % CPR;
            *reinterpret_cast<u32x4 *>(&kt[buf * kTile + key * KP + 8 * e8]) = kreg[i];
            *reinterpret_cast<u32x4 *>(&kt[buf * kTile + KB * KP + key * VP + 8 * e8]) = vreg[i];
        }
    };

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);

    // per-lane element offsets into a tile: K rows for the first product, the transposing read of V for the second
    const int k_lane = ql * KP + 8 * g;
    const int v_lane = KB * KP + (4 * g + (ql >> 2)) * VP + 4 * (ql & 3);

    auto block = [&](int it, int buf, bool masked) {
        const uint16_t *tile = kt + buf * kTile;
        const int kb = it * KB;
        floatx4 s[NKK][2];
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            s[kk][0] = s[kk][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < HD / 32; ++ks) {
                const bf16x8 a = *reinterpret_cast<const bf16x8 *>(&tile[k_lane + 16 * kk * KP + 32 * ks]);
                s[kk][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[0][ks], s[kk][0], 0, 0, 0);
                s[kk][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[1][ks], s[kk][1], 0, 0, 0);
            }
        }
        // s[kk][b][r] is the raw score of key kb + 16 kk + 4 g + r against query qi[b]
        bf16x8 pb[2][NT];   // [query block][K-step of 32 keys]
        float bm[2];
        bool lag = false;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if (masked) {   // (wave-uniform; one copy of the products for both cases keeps the output registers in place)
#pragma unroll
                for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (kb + 16 * kk + 4 * g + r > qi[b]) s[kk][b][r] = kMasked;
            }
            float v = fmaxf(s[0][b][0], s[0][b][1]);
            v = fmaxf(fmaxf(v, s[0][b][2]), s[0][b][3]);
#pragma unroll
            for (int kk = 1; kk < NKK; ++kk) {
                v = fmaxf(fmaxf(v, s[kk][b][0]), s[kk][b][1]);
                v = fmaxf(fmaxf(v, s[kk][b][2]), s[kk][b][3]);
            }
            bm[b] = max_over_lane_groups(v);
            lag = lag || (bm[b] - m[b]) * p.scale_log2 > kLazy;
        }
        // The reference maximum follows the true one only when that has moved by more than 2^kLazy (probabilities up to
        // 2^kLazy instead of 1: harmless in fp32 and bf16, and the final division takes the factor out again), so the
        // rescaling of the 2 (HD / 16 + 1) accumulators is rare after the first blocks.  (The first block always
        // rescales: finite against -1e30; key 0 is visible to every query.)
        if (__builtin_amdgcn_ballot_w64(lag) != 0) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const float m_new = fmaxf(m[b], bm[b]);
                const float alpha = __builtin_amdgcn_exp2f((m[b] - m_new) * p.scale_log2);
                m[b] = m_new;
                l[b] *= alpha;
#pragma unroll
                for (int d = 0; d < HD / 16; ++d) o[b][d] *= alpha;
            }
        }
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const float msc = m[b] * p.scale_log2;
            // v_exp_f32 directly: results that would be denormal may flush to zero, and a masked score (-1e30 against a
            // finite maximum) gives exactly 0
#pragma unroll
            for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
                for (int r = 0; r < 4; ++r) s[kk][b][r] = __builtin_amdgcn_exp2f(fmaf(s[kk][b][r], p.scale_log2, -msc));
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                u32x4 pw;
                pw[0] = pack_bf16x2(s[2 * t][b][0], s[2 * t][b][1]);
                pw[1] = pack_bf16x2(s[2 * t][b][2], s[2 * t][b][3]);
                pw[2] = pack_bf16x2(s[2 * t + 1][b][0], s[2 * t + 1][b][1]);
                pw[3] = pack_bf16x2(s[2 * t + 1][b][2], s[2 * t + 1][b][3]);
                pb[b][t] = __builtin_bit_cast(bf16x8, pw);
                l[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[b][t], l[b], 0, 0, 0);
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int d = 0; d < HD / 16; ++d) {
                const uint16_t *src = &tile[v_lane + 32 * t * VP + 16 * d];
                const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *)src);
                const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *)(src + 16 * VP));
                const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
                const u32x4 aw = {lo2.x, lo2.y, hi2.x, hi2.y};
                const bf16x8 a = __builtin_bit_cast(bf16x8, aw);
                o[0][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[0][t], o[0][d], 0, 0, 0);
                o[1][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[1][t], o[1][d], 0, 0, 0);
            }
    };

    // Every wave of the workgroup runs hA steps with one barrier each (set 1 may have one step less to do).  Step s
    // multiplies from buffer s % 2, filled at the head of step s - 1 from registers loaded during step s - 2.
    // Set 1's change of item sits between two copies of the step loop, not inside one: a loop that may reload the
    // queries makes the compiler wait for the block in flight before the first MFMA of every step, and copy the
    // output registers around the reset.
    auto steps = [&](int s_begin, int s_end) {
        for (int s = s_begin; s < s_end; ++s) {
            const int buf = s & 1;
            if (block_of_step(s + 1) >= 0) {
                stage(buf ^ 1);                  // read last during step s - 1, before the barrier that ended it
                if (block_of_step(s + 2) >= 0) fetch(block_of_step(s + 2));
            }
            const int it = block_of_step(s);
            const int kb = it * KB;
            if (it >= 0 && kb <= q0 + 31) block(it, buf, kb + KB - 1 > q0);   // else every key is after this wave's queries
            __syncthreads();
        }
    };
    const bool own_item = set == 1 && nB > 0;    // set 1 starts on the light item
    begin_item(own_item ? xb : xa);
    if (block_of_step(0) >= 0) {
        fetch(block_of_step(0));
        stage(0);
    }
    if (block_of_step(1) >= 0) fetch(block_of_step(1));
    __syncthreads();
    const int s_switch = own_item ? nB : hA;     // nB <= hA
    steps(0, s_switch);
    if (own_item) {                              // set 1 goes over to the heavy item's last blocks
        store_item();
        begin_item(xa);
    }
    steps(s_switch, hA);

    // Set 1's partial result for the heavy item (neutral if it had no block of it) goes through LDS, lane to lane: the
    // same wave and lane of set 0 owns the same queries and output elements.
    constexpr int NREG = 2 * (HD / 16) * 4 + 4;
    float *xch = reinterpret_cast<float *>(attn_lds) + w4 * NREG * 64 + lane;
    if (set == 1) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int d = 0; d < HD / 16; ++d)
#pragma unroll
                for (int r = 0; r < 4; ++r) xch[((b * (HD / 16) + d) * 4 + r) * 64] = o[b][d][r];
            xch[(NREG - 4 + b) * 64] = m[b];
            xch[(NREG - 2 + b) * 64] = l[b][0];
        }
    }
    __syncthreads();
    if (set == 1) return;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const float m1 = xch[(NREG - 4 + b) * 64], l1 = xch[(NREG - 2 + b) * 64];
        const float mm = fmaxf(m[b], m1);
        const float f0 = __builtin_amdgcn_exp2f((m[b] - mm) * p.scale_log2), f1 = __builtin_amdgcn_exp2f((m1 - mm) * p.scale_log2);
        l[b][0] = l[b][0] * f0 + l1 * f1;
#pragma unroll
        for (int d = 0; d < HD / 16; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[b][d][r] = o[b][d][r] * f0 + xch[((b * (HD / 16) + d) * 4 + r) * 64] * f1;
    }
    store_item();
}

template <int HD, int HPW>
hipError_t launch_attn(const PrefillAttnParams &p, hipStream_t stream) {
    constexpr size_t lds = attn_lds_bytes<HD>();
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&prefill_attn_kernel<HD, HPW>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    constexpr int QW = 32 * (4 / HPW);
    const int nx = (p.M + QW - 1) / QW;
    const dim3 grid((nx + 1) / 2, p.n_kv * (p.n_heads / p.n_kv / HPW));
    hipLaunchKernelGGL((prefill_attn_kernel<HD, HPW>), grid, dim3(512), lds, stream, p);
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
