// Final RMSNorm + bf16 lm_head GEMV + argmax for gfx950: the tail of a decode step
// (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_inference.py:459-486).
//
//     normed = bf16((x / sqrt(mean(x^2) + eps)) * norm_w)        fp32, the host rms_norm of the reference
//     logits[v] = bf16(sum_e W[v, e] * normed[e])                W bf16 [V, E] row-major, fp32 accumulation
//     argmax = first index of the largest logit                   (np.argmax over the bf16 logits)
//
// HBM-bound: every byte of W (2 V E, 525 MB for the 1B model) is read once.  A wavefront owns 16
// consecutive rows; the normalised x lives in registers as packed bf16 pairs (E / 64 values per lane),
// a row is read as E / 512 fully coalesced 1 KiB wave loads, and v_dot2c_f32_bf16 does two
// multiply-adds per 32-bit word (exact bf16 x bf16 products, fp32 sum).  The rows of a group are
// reduced over the 64 lanes by a butterfly; lane r keeps row r's sum, so the wave's 16 logits leave
// as one 32-byte store.  Each wave also writes max((orderable logit << 32) | ~row) for its rows; a
// one-workgroup kernel reduces those keys to the argmax (largest logit, lowest row on ties).
#include "common.h"
#include "kernels.h"

namespace w4a16 {

namespace {

#ifndef LM_RPW
#define LM_RPW 16
#endif
#ifndef LM_WAVES
#define LM_WAVES 4
#endif
#ifndef LM_RG
#define LM_RG 4
#endif
#ifndef LM_NT
#define LM_NT 1
#endif
constexpr int kRowsPerWave = LM_RPW;
constexpr int kWaves = LM_WAVES;

struct LmHeadParams {
    const uint16_t *x;
    const uint16_t *norm_w;   // nullptr: x is used as it is
    float eps;
    const uint16_t *w;
    uint16_t *logits;
    unsigned long long *keys;   // one per wave
    int V, E;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

__device__ __forceinline__ unsigned long long wave_max(unsigned long long v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const unsigned long long o = __shfl_xor(v, m, 64);
        v = o > v ? o : v;
    }
    return v;
}

// By value on purpose: __builtin_bit_cast applied directly to an element of an ext_vector reads element 0
// whatever the index (hipcc 7.2), so the element is copied into a scalar first.
__device__ __forceinline__ bf16x2 as_bf16x2(uint32_t v) { return __builtin_bit_cast(bf16x2, v); }

// bf16 bit pattern -> unsigned key with the same order as the value (-0 counts as +0).
__device__ __forceinline__ uint32_t orderable(uint32_t bits16) {
    if (bits16 == 0x8000u) bits16 = 0;
    return (bits16 & 0x8000u) ? (~bits16 & 0xFFFFu) : (bits16 | 0x8000u);
}

// NCH 16-byte chunks per lane and row (512 NCH >= E); RG rows are loaded together.  RAGGED: E is not
// 512 NCH, lanes past the end of a row load nothing and contribute zeros.
template <int NCH, int RG, bool RAGGED>
__global__ void __launch_bounds__(kWaves * 64) lm_head_kernel(const LmHeadParams p) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const int row0 = gw * kRowsPerWave;
    if (row0 >= p.V) return;                         // whole waves leave; the kernel has no barrier

    // chunk c of a row covers elements 512 c + 8 lane .. + 7
    u32x4 xp[NCH];
    bool in_row[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        in_row[c] = !RAGGED || 512 * c + 8 * lane < p.E;
        xp[c] = u32x4{0u, 0u, 0u, 0u};
        if (in_row[c]) xp[c] = *reinterpret_cast<const u32x4 *>(p.x + 512 * c + 8 * lane);
    }
    if (p.norm_w) {
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < NCH; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = bf16_bits_to_float(xp[c][e] & 0xFFFFu), hi = bf16_bits_to_float(xp[c][e] >> 16);
                ss = fmaf(lo, lo, ss);
                ss = fmaf(hi, hi, ss);
            }
        const float rms = sqrtf(wave_sum(ss) / (float)p.E + p.eps);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            u32x4 nw = u32x4{0u, 0u, 0u, 0u};
            if (in_row[c]) nw = *reinterpret_cast<const u32x4 *>(p.norm_w + 512 * c + 8 * lane);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = bf16_bits_to_float(xp[c][e] & 0xFFFFu), hi = bf16_bits_to_float(xp[c][e] >> 16);
                const float wl = bf16_bits_to_float(nw[e] & 0xFFFFu), wh = bf16_bits_to_float(nw[e] >> 16);
                xp[c][e] = pack_bf16x2((lo / rms) * wl, (hi / rms) * wh);
            }
        }
    }

    float mine = 0.f;
    const size_t row_words = (size_t)p.E / 8;        // u32x4 per row
    const u32x4 *wbase = reinterpret_cast<const u32x4 *>(p.w) + lane;
#pragma unroll
    for (int r = 0; r < kRowsPerWave; r += RG) {
        u32x4 wv[RG][NCH];
#pragma unroll
        for (int i = 0; i < RG; ++i) {
            int row = row0 + r + i;
            row = row < p.V ? row : p.V - 1;         // ragged V: load in range, never stored
            const u32x4 *src = wbase + (size_t)row * row_words;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                wv[i][c] = u32x4{0u, 0u, 0u, 0u};
                if (in_row[c]) wv[i][c] = LM_NT ? __builtin_nontemporal_load(src + 64 * c) : src[64 * c];
            }
        }
#pragma unroll
        for (int i = 0; i < RG; ++i) {
            float a0 = 0.f, a1 = 0.f;                // two chains: the dot instruction accumulates in place
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                a0 = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(wv[i][c][0]), as_bf16x2(xp[c][0]), a0, false);
                a1 = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(wv[i][c][1]), as_bf16x2(xp[c][1]), a1, false);
                a0 = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(wv[i][c][2]), as_bf16x2(xp[c][2]), a0, false);
                a1 = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(wv[i][c][3]), as_bf16x2(xp[c][3]), a1, false);
            }
            const float s = wave_sum(a0 + a1);
            mine = lane == r + i ? s : mine;
        }
    }

    const int row = row0 + lane;
    const bool valid = lane < kRowsPerWave && row < p.V;
    const uint32_t bits = float_to_bf16_bits(mine);
    if (valid) p.logits[row] = (uint16_t)bits;
    unsigned long long key = 0;
    if (valid) key = ((unsigned long long)orderable(bits) << 32) | (0xFFFFFFFFu - (uint32_t)row);
    key = wave_max(key);
    if (lane == 0) p.keys[gw] = key;
}

__global__ void __launch_bounds__(1024) lm_head_argmax_kernel(const unsigned long long *keys, int n, int32_t *out) {
    __shared__ unsigned long long part[16];
    unsigned long long best = 0;
    // eight independent loads per thread and round trip (one round for up to 131072 rows)
    for (int base = 0; base < n; base += 8 * 1024) {
        unsigned long long k[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = base + j * 1024 + (int)threadIdx.x;
            k[j] = i < n ? keys[i] : 0ull;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) best = k[j] > best ? k[j] : best;
    }
    best = wave_max(best);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 1; i < 16; ++i) best = part[i] > best ? part[i] : best;
        out[0] = (int32_t)(0xFFFFFFFFu - (uint32_t)(best & 0xFFFFFFFFull));
    }
}

template <int NCH, int RG>
void launch_one(const LmHeadParams &p, int grid, hipStream_t stream) {
    if (p.E == 512 * NCH)
        hipLaunchKernelGGL((lm_head_kernel<NCH, RG, false>), dim3(grid), dim3(kWaves * 64), 0, stream, p);
    else
        hipLaunchKernelGGL((lm_head_kernel<NCH, RG, true>), dim3(grid), dim3(kWaves * 64), 0, stream, p);
}

// Smallest instantiated chunk count that covers E, 0 if there is none.
int chunks_for(int E) {
    const int need = (E + 511) / 512;
    for (int nch : {1, 2, 3, 4, 6, 8, 10, 12, 16})
        if (nch >= need) return nch;
    return 0;
}

}  // namespace

bool lm_head_supported(int V, int E) { return V > 0 && E > 0 && E % 8 == 0 && chunks_for(E) != 0; }

size_t lm_head_scratch_bytes(int V) {
    const size_t waves = ((size_t)V + kRowsPerWave - 1) / kRowsPerWave;
    return ((waves * sizeof(unsigned long long) + 255) / 256) * 256;
}

hipError_t launch_lm_head(const uint16_t *x, const uint16_t *norm_w, float eps, const uint16_t *w, uint16_t *logits,
                          int32_t *argmax_out, int V, int E, void *workspace, hipStream_t stream) {
    LmHeadParams p;
    p.x = x;
    p.norm_w = norm_w;
    p.eps = eps;
    p.w = w;
    p.logits = logits;
    p.keys = static_cast<unsigned long long *>(workspace);
    p.V = V;
    p.E = E;
    const int waves = (V + kRowsPerWave - 1) / kRowsPerWave;
    const int grid = (waves + kWaves - 1) / kWaves;
    switch (chunks_for(E)) {
        case 1: launch_one<1, 4>(p, grid, stream); break;
        case 2: launch_one<2, 4>(p, grid, stream); break;
        case 3: launch_one<3, 4>(p, grid, stream); break;
        case 4: launch_one<4, LM_RG>(p, grid, stream); break;
        case 6: launch_one<6, 2>(p, grid, stream); break;
        case 8: launch_one<8, 2>(p, grid, stream); break;
        case 10: launch_one<10, 1>(p, grid, stream); break;
        case 12: launch_one<12, 1>(p, grid, stream); break;
        case 16: launch_one<16, 1>(p, grid, stream); break;
        default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !argmax_out) return e;
    hipLaunchKernelGGL(lm_head_argmax_kernel, dim3(1), dim3(1024), 0, stream, p.keys, waves, argmax_out);
    return hipGetLastError();
}

}  // namespace w4a16
