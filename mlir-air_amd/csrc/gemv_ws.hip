// Whole-K decode GEMV on the stream-order layout (wstream.h), M = 1, and the re-pack kernel that
// writes that layout from the AutoAWQ checkpoint tensors.
//
// HBM-bound: every packed byte is read once, as 1 KiB global_load_dwordx4 wave loads.  A workgroup
// owns one 16-column tile for all of K and writes its 16 outputs itself: no partial sums leave the
// workgroup, so there is no workspace, no cross-workgroup protocol and no state between calls.
//
// Arithmetic on the matrix cores (the fp32 VALU cannot keep up with HBM: ~2.5 lane-ops per weight
// at 8 TB/s, a convert + FMA needs ~2.4; building an MFMA operand costs 7 ops per 8 weights).
//
// Launch-shape notes (K = 4096, N = 11008, cold): tasks of 8 cells with one wave each (4 waves per tile) 5.9 us,
// 16 cells 6.3 us, 4 cells 5.9 us, fewer waves than tasks 6.3-6.8 us.  Tried and not kept: the four K-steps of a
// cell as four independent MFMAs on an A operand of 4 groups x 4 K-steps (one coalesced x load per four cells instead
// of four strided ones): the adds of the four results wait out the MFMA latency, 6.1 us; cells in interleaved pairs:
// 6.0 us; x fetched with coalesced loads and brought into operand order through wave-local LDS rows: 5.9 us, no gain.
//
//   task   = up to CT consecutive groups of one block of one tile: all its loads (4 of x, CT cells,
//            1 of scales / zero points) are issued before anything is consumed, cells are
//            consumed in arrival order
//   wave   = tasks w, w + W, ... of the tile's NB * (16 / CT) tasks (W waves per workgroup)
//
// M = 1 uses one of the 16 rows of an MFMA product.  Instead of broadcasting x to all rows, row r
// of the A operand holds the x values of group r of the block (one coalesced load per K-step: lane
// (lg, ln) reads x[128 (16 b + ln) + 32 t + 8 lg ..+7]).  The product with the cell of group r0 is
// then wanted in row r0 only; the other rows multiply x of one group with weights of another and
// are never read.  Row r0 lives in register r0 % 4 of lane group r0 / 4, which is exactly where the
// block's scales and zero points of group r0 were loaded (wstream.h), and where the ones-product
// sum_k x[k] of group r0 lands.  So after the 16 cells of a block each lane flushes four groups:
//        y += s * (sum (128 + q) x  -  (128 + z) * sum x)
// with 0x4300 | q == bf16(128 + q) exactly, and the lanes of a column are added up at the end.
#include <algorithm>

#include "common.h"
#include "kernels.h"
#include "wstream.h"

namespace w4a16 {

namespace {

constexpr int kMaxWaves = 16;

// (dword >> 4 v) & 0x000F000F | 0x43004300: rows (2 v, 2 v + 1) of the lane's column as bf16 (128 + q)
__device__ __forceinline__ bf16x8 cell_operand(uint32_t w, uint32_t nib_mask, uint32_t magic) {
    u32x4 b;
#pragma unroll
    for (int v = 0; v < 4; ++v) b[v] = ((w >> (4 * v)) & nib_mask) | magic;
    return __builtin_bit_cast(bf16x8, b);
}

// Arguments that only some launches read; they follow the ones every wave needs at once, which fit the SGPRs
// that arrive with the wave.
struct GemvWsTail {
    const uint16_t *norm_w;    // RMS: bf16 [K]
    const float *sumsq_in;     // RMS: partial sums of x^2 left by the launch that produced x, or null (the wave walks x)
    float *sumsq_out;          // sum of squares of this launch's bf16 outputs, one float per 16-column tile, or null
    float eps;
    int sumsq_n;
    int K;
};

// a0 += sum of squares of the low bf16 halves of v, a1 += of the high halves
__device__ __forceinline__ void sumsq8(const u32x4 v, float &a0, float &a1) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = __builtin_bit_cast(float, v[j] << 16);
        const float hi = __builtin_bit_cast(float, v[j] & 0xFFFF0000u);
        a0 = fmaf(lo, lo, a0);
        a1 = fmaf(hi, hi, a1);
    }
}

// CT   cells per task (4, 8 or 16)
// NMAT 1, or 2: gate and up matrices with the SwiGLU epilogue h = bf16(silu(bf16 g) * bf16 u)
// RMS  x is RMS-normalised on the fly: every wave obtains rstd = 1 / sqrt(mean(x^2) + eps) itself (from the partial
//      sums the producer of x left behind, else by walking x, which is K bf16 values and L2-resident) and feeds
//      bf16((x * rstd) * norm_w) to the matrix cores
// Q4   Q4NX order: a scale and a min per K-step of a cell; the four K-steps of a cell are four products of their own and
//      the flush is y += s (sum (128 + q) x - 128 sum x) + min' sum x per K-step
template <int CT, int NMAT, bool RMS, bool Q4>
__global__ void __launch_bounds__(kMaxWaves * 64) gemv_ws_kernel(const uint16_t *__restrict__ x, const char *__restrict__ w0,
                                                                 const char *__restrict__ w1, uint16_t *__restrict__ y,
                                                                 const uint16_t *__restrict__ residual, int G, int NB,
                                                                 int round_before_add, int nwaves, const GemvWsTail tail) {
    constexpr int SUB = kWsBlockGroups / CT;
    __shared__ float red[NMAT * kMaxWaves * kWsTileCols];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    const int tile = blockIdx.x;
    constexpr int MDK = Q4 ? kWsQ4MdKiB : 1;   // KiB of scale words in front of a block's cells
    const size_t tile_bytes = (size_t)(MDK * NB + G) * kWsCellBytes;

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
    // Kept opaque so that (v & mask) | magic stays one v_and_or_b32 with register operands.
    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));

    float yv[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) yv[m] = 0.f;

    // RMS: the partial sums are requested first and consumed only after the first task's loads have been requested
    // (below), so that their round trip overlaps with the weights' instead of standing in front of them (gate / up
    // launch of the decode block: 17.3 -> 12.9 us).
    float rstd = 0.f, a0 = 0.f, a1 = 0.f;
    float piece[4] = {0.f, 0.f, 0.f, 0.f};
    bool have_rstd = !RMS;
    if constexpr (RMS) {
        if (tail.sumsq_in && tail.sumsq_n <= 256) {
#pragma unroll
            for (int i = 0; i < 4; ++i) piece[i] = lane + 64 * i < tail.sumsq_n ? tail.sumsq_in[lane + 64 * i] : 0.f;
        } else if (tail.sumsq_in) {
            for (int i = lane; i < tail.sumsq_n; i += 64) a0 += tail.sumsq_in[i];
        } else {
            const u32x4 *xv = reinterpret_cast<const u32x4 *>(x);
            const int nchunks = tail.K >> 3;
            for (int c0 = lane; c0 < nchunks; c0 += 512) {   // 8 loads in flight
                u32x4 v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = c0 + 64 * i < nchunks ? xv[c0 + 64 * i] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int i = 0; i < 8; ++i) sumsq8(v[i], a0, a1);
            }
        }
    }

    const int tasks_per_mat = NB * SUB;
    for (int task = wave; task < NMAT * tasks_per_mat; task += nwaves) {
        const int mat = NMAT == 1 ? 0 : task / tasks_per_mat;
        const int tm = task - mat * tasks_per_mat;
        const int b = tm / SUB, r0 = (tm % SUB) * CT;
        const int ng = min(kWsBlockGroups, G - kWsBlockGroups * b);   // groups of this block
        if (r0 >= ng) continue;                                       // wave-uniform
        const char *blk = (mat ? w1 : w0) + (size_t)tile * tile_bytes + (size_t)b * ((kWsBlockGroups + MDK) * kWsCellBytes);

        // x of the task's groups: A row ln <-> group 16 b + ln; rows outside the task are zero, so that
        // their (never read) products and their sum x stay finite and contribute nothing
        const int grow = kWsBlockGroups * b + ln;
        const bool xvalid = ln >= r0 && ln < r0 + CT && grow < G;
        const uint16_t *xp = x + (size_t)(xvalid ? grow : 0) * 128 + 8 * lg;
        u32x4 X[4], cell[CT];
        u32x4 NW[RMS ? 4 : 1];
#pragma unroll
        for (int t = 0; t < 4; ++t) X[t] = *reinterpret_cast<const u32x4 *>(xp + 32 * t);
        if constexpr (RMS) {
            const uint16_t *np = tail.norm_w + (size_t)(xvalid ? grow : 0) * 128 + 8 * lg;
#pragma unroll
            for (int t = 0; t < 4; ++t) NW[t] = *reinterpret_cast<const u32x4 *>(np + 32 * t);
        }
        // scales / zero points next: they sit right in front of the cells (requested after the cells instead: +0.5 us)
        u32x4 md[MDK];
#pragma unroll
        for (int t = 0; t < MDK; ++t) md[t] = *(reinterpret_cast<const u32x4 *>(blk + (size_t)t * kWsCellBytes) + lane);
#pragma unroll
        for (int r = 0; r < CT; ++r) {
            const int rc = r0 + r < ng ? r0 + r : ng - 1;   // a short block re-reads its last cell (x of that row is zero)
            cell[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(blk + (size_t)(MDK + rc) * kWsCellBytes) + lane);
        }
        // every load of the task is requested before the first wait
        __builtin_amdgcn_sched_barrier(0);

        if constexpr (RMS) {
            if (!have_rstd) {   // wave-uniform; the pieces are added in the order a lane walking them would
                // (taken opaque here: the sum does not depend on the loop, and hoisted in front of it the wait for the
                // pieces would stand before the task's requests after all)
                asm volatile("" : "+v"(piece[0]), "+v"(piece[1]), "+v"(piece[2]), "+v"(piece[3]), "+v"(a0), "+v"(a1));
                a0 += ((piece[0] + piece[1]) + piece[2]) + piece[3];
                rstd = 1.0f / sqrtf(wave_reduce<false>(a0 + a1) / (float)tail.K + tail.eps);
                have_rstd = true;
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float x_lo = __builtin_bit_cast(float, X[t][j] << 16), x_hi = __builtin_bit_cast(float, X[t][j] & 0xFFFF0000u);
                    const float w_lo = __builtin_bit_cast(float, NW[t][j] << 16), w_hi = __builtin_bit_cast(float, NW[t][j] & 0xFFFF0000u);
                    X[t][j] = pack_bf16x2((x_lo * rstd) * w_lo, (x_hi * rstd) * w_hi);
                }
            }
        }
        if (!xvalid) {
#pragma unroll
            for (int t = 0; t < 4; ++t) X[t] = u32x4{0u, 0u, 0u, 0u};
        }
        float sum = 0.f;
        if constexpr (!Q4) {
            floatx4 xs = {0.f, 0.f, 0.f, 0.f};   // register i of lane group lg: sum of x over group 16 b + 4 lg + i
#pragma unroll
            for (int t = 0; t < 4; ++t) xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[t]), ones, xs, 0, 0, 0);

            float V[4] = {0.f, 0.f, 0.f, 0.f};   // V[i] of lane group lg: sum (128 + q) x of group 16 b + 4 lg + i
#pragma unroll
            for (int r = 0; r < CT; ++r) {
                floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[t]), cell_operand(cell[r][t], nib_mask, magic),
                                                                  acc, 0, 0, 0);
                V[r & 3] = (lg == ((r0 + r) >> 2)) ? acc[r & 3] : V[r & 3];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float s = __builtin_bit_cast(float, md[0][i] << 16);
                const float nz = __builtin_bit_cast(float, md[0][i] & 0xFFFF0000u);   // -(128 + z)
                sum = fmaf(s, fmaf(nz, xs[i], V[i]), sum);
            }
        } else {
            const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
            floatx4 xs[4];                        // xs[t][i]: sum of x over rows 32 t .. 32 t + 31 of group 16 b + 4 lg + i
#pragma unroll
            for (int t = 0; t < 4; ++t) xs[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[t]), ones, zero4, 0, 0, 0);
            float V[4][4];                        // V[t][i]: sum (128 + q) x over the same rows
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) V[t][i] = 0.f;
#pragma unroll
            for (int r = 0; r < CT; ++r) {
                const bool mine = lg == ((r0 + r) >> 2);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const floatx4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[t]),
                                                                                cell_operand(cell[r][t], nib_mask, magic), zero4, 0, 0, 0);
                    V[t][r & 3] = mine ? acc[r & 3] : V[t][r & 3];
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float s = __builtin_bit_cast(float, md[t][i] << 16);
                    const float mn = __builtin_bit_cast(float, md[t][i] & 0xFFFF0000u);
                    sum = fmaf(s, fmaf(-128.0f, xs[t][i], V[t][i]), fmaf(mn, xs[t][i], sum));
                }
        }
        if (NMAT == 2 && mat) yv[NMAT - 1] += sum;
        else yv[0] += sum;
    }

    // K-reduction: the 4 lane groups of a wave hold different groups of K for the same 16 columns and are added with
    // wavefront shuffles, (lg 0 + lg 1) + (lg 2 + lg 3); only the waves' sums meet in LDS, added by the first 16 threads
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
        float v = yv[m];
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        if (lg == 0) red[(m * kMaxWaves + wave) * kWsTileCols + ln] = v;
    }
    __syncthreads();
    if (threadIdx.x < kWsTileCols) {
        float tot[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            tot[m] = 0.f;
            for (int w = 0; w < nwaves; ++w) tot[m] += red[(m * kMaxWaves + w) * kWsTileCols + threadIdx.x];
        }
        const int col = tile * kWsTileCols + threadIdx.x;
        float out;
        if (NMAT == 2) {
            const float gate = bf16_bits_to_float(float_to_bf16_bits(tot[0]));
            const float up = bf16_bits_to_float(float_to_bf16_bits(tot[NMAT - 1]));
            out = silu_tanh(gate) * up;
        } else {
            out = tot[0];
        }
        if (residual) {
            if (round_before_add) out = bf16_bits_to_float(float_to_bf16_bits(out));
            out += bf16_bits_to_float(residual[col]);
        }
        const uint16_t ob = float_to_bf16_bits(out);
        y[col] = ob;
        if (tail.sumsq_out) {   // the 16 outputs of the tile as the next RMSNorm will read them
            const float r = bf16_bits_to_float(ob);
            float sq = r * r;
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
            if (threadIdx.x == 0) tail.sumsq_out[tile] = sq;
        }
    }
}

// Read-only pass over a stream-order matrix with the GEMV's launch shape and request pattern (one workgroup per tile,
// a wave per task of CT cells, the block's scale words and the cells requested up front, non-temporal cell loads):
// everything loaded is folded with XOR into one word per wave.  No x, no arithmetic: what this takes is the floor of
// any kernel that reads the buffer once in this order.
template <int CT>
__global__ void __launch_bounds__(kMaxWaves * 64) probe_ws_kernel(const char *__restrict__ w, uint32_t *__restrict__ out, int G, int NB,
                                                                  int nwaves) {
    constexpr int SUB = kWsBlockGroups / CT;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const size_t tile_bytes = (size_t)(NB + G) * kWsCellBytes;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (int task = wave; task < NB * SUB; task += nwaves) {
        const int b = task / SUB, r0 = (task % SUB) * CT;
        const int ng = min(kWsBlockGroups, G - kWsBlockGroups * b);
        if (r0 >= ng) continue;
        const char *blk = w + (size_t)blockIdx.x * tile_bytes + (size_t)b * ((kWsBlockGroups + 1) * kWsCellBytes);
        u32x4 cell[CT];
        const u32x4 md = *(reinterpret_cast<const u32x4 *>(blk) + lane);
#pragma unroll
        for (int r = 0; r < CT; ++r) {
            const int rc = r0 + r < ng ? r0 + r : ng - 1;
            cell[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(blk + (size_t)(1 + rc) * kWsCellBytes) + lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        acc ^= md;
#pragma unroll
        for (int r = 0; r < CT; ++r) acc ^= cell[r];
    }
    uint32_t v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off);
    if (lane == 0) out[blockIdx.x * kMaxWaves + wave] = v;
}

// One thread per dword of the stream-order buffer.
__global__ void __launch_bounds__(256) repack_ws_kernel(const uint32_t *__restrict__ qweight, const uint32_t *__restrict__ qzeros,
                                                        const uint16_t *__restrict__ scales, uint32_t *__restrict__ out, int G,
                                                        int NB, int N) {
    const size_t tile_dwords = (size_t)(NB + G) * (kWsCellBytes / 4);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= tile_dwords * (N / kWsTileCols)) return;
    const int tile = (int)(idx / tile_dwords);
    const int off = (int)(idx - (size_t)tile * tile_dwords);
    constexpr int BLOCK_DWORDS = (kWsBlockGroups + 1) * (int)(kWsCellBytes / 4);
    const int b = min(off / BLOCK_DWORDS, NB - 1);
    const int within = off - b * BLOCK_DWORDS;
    const int l = (within & 255) >> 2, sub = within & 3;   // lane and dword of a 1 KiB piece
    const int n = tile * kWsTileCols + (l & 15);
    const int lg = l >> 4;
    const int nb = N >> 3;
    const int shift = 4 * unpack_pos(n & 7);               // where column n sits in its checkpoint word
    uint32_t v = 0;
    if (within < 256) {                                    // scales and zero points
        const int g = kWsBlockGroups * b + 4 * lg + sub;
        if (g < G) {
            const uint32_t z = (qzeros[(size_t)g * nb + (n >> 3)] >> shift) & 0xFu;
            v = (uint32_t)scales[(size_t)g * N + n] | ((0xC300u | z) << 16);
        }
    } else {
        const int g = kWsBlockGroups * b + (within >> 8) - 1;
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int k = 128 * g + 32 * sub + 8 * lg + pack_order(p);
            v |= ((qweight[(size_t)k * nb + (n >> 3)] >> shift) & 0xFu) << (4 * p);
        }
    }
    out[idx] = v;
}

// Q4NX order from the operands of the affine path; one thread per dword of the buffer.
__global__ void __launch_bounds__(256) repack_ws_q4_kernel(const uint32_t *__restrict__ qweight, const uint16_t *__restrict__ scales,
                                                           const uint16_t *__restrict__ mins, uint32_t *__restrict__ out, int G, int NB,
                                                           int N) {
    const size_t tile_dwords = (size_t)(kWsQ4MdKiB * NB + G) * (kWsCellBytes / 4);
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= tile_dwords * (N / kWsTileCols)) return;
    const int tile = (int)(idx / tile_dwords);
    const int off = (int)(idx - (size_t)tile * tile_dwords);
    constexpr int BLOCK_DWORDS = (kWsBlockGroups + kWsQ4MdKiB) * (int)(kWsCellBytes / 4);
    const int b = min(off / BLOCK_DWORDS, NB - 1);
    const int within = off - b * BLOCK_DWORDS;
    const int l = (within & 255) >> 2, sub = within & 3;   // lane and dword of a 1 KiB piece
    const int n = tile * kWsTileCols + (l & 15);
    const int lg = l >> 4;
    const int nb = N >> 3;
    const int shift = 4 * unpack_pos(n & 7);               // where column n sits in its packed word
    uint32_t v = 0;
    if (within < kWsQ4MdKiB * 256) {                       // scales and mins: KiB t, dword i = group 16 b + 4 lg + i
        const int t = within >> 8;
        const int g = kWsBlockGroups * b + 4 * lg + sub;
        if (g < G) {
            const size_t at = (size_t)(4 * g + t) * N + n;
            v = (uint32_t)scales[at] | ((uint32_t)mins[at] << 16);
        }
    } else {
        const int g = kWsBlockGroups * b + (within >> 8) - kWsQ4MdKiB;
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int k = 128 * g + 32 * sub + 8 * lg + pack_order(p);
            v |= ((qweight[(size_t)k * nb + (n >> 3)] >> shift) & 0xFu) << (4 * p);
        }
    }
    out[idx] = v;
}

template <int CT>
hipError_t launch_ct(int nmat, int waves, const uint16_t *x, const void *w0, const void *w1, uint16_t *y, int K, int N,
                     const GemvWsExtras &ex, hipStream_t stream) {
    const int G = K / kGroup, NB = ws_blocks(K);
    const dim3 grid(N / kWsTileCols), block(waves * 64);
    const GemvWsTail tail = {ex.norm_w, ex.sumsq_in, ex.sumsq_out, ex.eps, ex.sumsq_n, K};
    const char *a = static_cast<const char *>(w0), *b = static_cast<const char *>(w1 ? w1 : w0);
#define W4A16_GEMV_WS_LAUNCH(NMAT, RMS, Q4)                                                                           \
    hipLaunchKernelGGL((gemv_ws_kernel<CT, NMAT, RMS, Q4>), grid, block, 0, stream, x, a, b, y, ex.residual, G, NB,  \
                       ex.round_before_add, waves, tail)
    if (ex.q4) {
        if constexpr (CT == 8) {   // (the Q4NX plan takes tasks of 8 cells only)
            if (ex.norm_w) {
                if (nmat == 2) W4A16_GEMV_WS_LAUNCH(2, true, true);
                else W4A16_GEMV_WS_LAUNCH(1, true, true);
            } else {
                if (nmat == 2) W4A16_GEMV_WS_LAUNCH(2, false, true);
                else W4A16_GEMV_WS_LAUNCH(1, false, true);
            }
        } else {
            return hipErrorInvalidValue;
        }
    } else if (ex.norm_w) {
        if (nmat == 2) W4A16_GEMV_WS_LAUNCH(2, true, false);
        else W4A16_GEMV_WS_LAUNCH(1, true, false);
    } else {
        if (nmat == 2) W4A16_GEMV_WS_LAUNCH(2, false, false);
        else W4A16_GEMV_WS_LAUNCH(1, false, false);
    }
#undef W4A16_GEMV_WS_LAUNCH
    return hipGetLastError();
}

}  // namespace

GemvWsTune g_gemv_ws_tune;

// Launch shape.  Tasks of 8 cells (16 tasks of a tile in flight at most); one wave per task up to 16 waves.
// A launch is fastest when all its waves are resident at once (every wave requests its whole task up front).  The
// RMSNorm variant needs 94 VGPRs at 8 cells per task, five waves per SIMD: a launch with more waves than that (gate +
// up of H = 14336: 7168) takes tasks of 16 cells instead, half as many waves of 124 VGPRs (block: 27.9 -> 26.9 us).
GemvWsPlan plan_gemv_ws(int K, int nmat, int N, bool rms) {
    GemvWsPlan pl;
    pl.ct = 8;
    if (rms && (long)(N / kWsTileCols) * std::min(nmat * ws_blocks(K) * (kWsBlockGroups / 8), kMaxWaves) > 5L * 4 * 256) pl.ct = 16;
    if (g_gemv_ws_tune.ct) pl.ct = g_gemv_ws_tune.ct;
    const int tasks = nmat * ws_blocks(K) * (kWsBlockGroups / pl.ct);
    pl.waves = tasks < kMaxWaves ? tasks : kMaxWaves;
    if (g_gemv_ws_tune.waves && g_gemv_ws_tune.waves < pl.waves) pl.waves = g_gemv_ws_tune.waves;
    return pl;
}

hipError_t launch_gemv_ws(const uint16_t *x, const void *w, const void *w_up, uint16_t *y, int K, int N, hipStream_t stream,
                          const GemvWsExtras &extras) {
    const int nmat = w_up ? 2 : 1;
    GemvWsPlan pl = plan_gemv_ws(K, nmat, N, extras.norm_w != nullptr);
    if (extras.q4 && pl.ct != 8) {   // Q4NX order: tasks of 8 cells
        pl.ct = 8;
        const int tasks = nmat * ws_blocks(K) * (kWsBlockGroups / 8);
        pl.waves = tasks < kMaxWaves ? tasks : kMaxWaves;
    }
    switch (pl.ct) {
        case 4: return launch_ct<4>(nmat, pl.waves, x, w, w_up, y, K, N, extras, stream);
        case 16: return launch_ct<16>(nmat, pl.waves, x, w, w_up, y, K, N, extras, stream);
        default: return launch_ct<8>(nmat, pl.waves, x, w, w_up, y, K, N, extras, stream);
    }
}

hipError_t launch_probe_ws(const void *w, uint32_t *out, int K, int N, hipStream_t stream) {
    const GemvWsPlan pl = plan_gemv_ws(K, 1, N, false);
    const int G = K / kGroup, NB = ws_blocks(K);
    const dim3 grid(N / kWsTileCols), block(pl.waves * 64);
    const char *p = static_cast<const char *>(w);
    if (pl.ct == 16) hipLaunchKernelGGL(probe_ws_kernel<16>, grid, block, 0, stream, p, out, G, NB, pl.waves);
    else if (pl.ct == 4) hipLaunchKernelGGL(probe_ws_kernel<4>, grid, block, 0, stream, p, out, G, NB, pl.waves);
    else hipLaunchKernelGGL(probe_ws_kernel<8>, grid, block, 0, stream, p, out, G, NB, pl.waves);
    return hipGetLastError();
}

hipError_t launch_repack_ws_q4(const int32_t *qweight, const uint16_t *scales, const uint16_t *mins, void *out, int K, int N,
                               hipStream_t stream) {
    const size_t dwords = ws_q4_matrix_bytes(K, N) / 4;
    const size_t blocks = (dwords + 255) / 256;
    if (blocks > 0x7FFFFFFFull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(repack_ws_q4_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<const uint32_t *>(qweight),
                       scales, mins, static_cast<uint32_t *>(out), K / kGroup, ws_blocks(K), N);
    return hipGetLastError();
}

hipError_t launch_repack_ws(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, void *out, int K, int N,
                            hipStream_t stream) {
    const size_t dwords = ws_matrix_bytes(K, N) / 4;
    const size_t blocks = (dwords + 255) / 256;
    if (blocks > 0x7FFFFFFFull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(repack_ws_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, reinterpret_cast<const uint32_t *>(qweight),
                       reinterpret_cast<const uint32_t *>(qzeros), scales, static_cast<uint32_t *>(out), K / kGroup, ws_blocks(K), N);
    return hipGetLastError();
}

}  // namespace w4a16

// ---- batched decode, 2 <= M <= 16 (gemm_ws_kernel) and up to 64 rows (gemm_ws_rows_kernel), on the same layout ----
//
// The 16 rows of the A operand are the rows of x (row m <-> lane ln = m), so a cell's product is the whole
// [16 x 16] block of y for its 16 columns and the group flush applies to all four accumulator registers.  A workgroup
// owns CB adjacent tiles (16 CB columns) for all of K, so that the x operands of a group (four gathered loads of
// 16 rows x 64 bytes) are built once for CB cells; its waves take the groups round-robin, four groups per task with
// every load of the task (16 of x, 4 CB cells, 4 CB scale words) requested up front.  The waves' [16 x 16 CB] partial
// sums meet in LDS and leave as bf16.  No workspace, nothing exchanged between workgroups.
namespace w4a16 {
namespace {

constexpr int kGemmWsWaves = 8;
constexpr int kGemmWsGroups = 4;   // groups per task

// Q4: the matrix is in Q4NX order (a scale and a min per 32 rows): every K-step of a cell is a product of its own,
// folded in at once as y += s sum((128 + q) x) + (min - 128 s) sum(x).
template <int CB, bool Q4>
__global__ void __launch_bounds__(kGemmWsWaves * 64) gemm_ws_kernel(const uint16_t *__restrict__ x, const char *__restrict__ w,
                                                                    uint16_t *__restrict__ y, const uint16_t *__restrict__ residual,
                                                                    int M, int K, int N, int G, int NB) {
    extern __shared__ __attribute__((aligned(16))) float red[];   // [wave][cb][reg][lane]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    constexpr int MDK = Q4 ? kWsQ4MdKiB : 1;   // KiB of scale words in front of a block's cells
    const size_t tile_bytes = (size_t)(MDK * NB + G) * kWsCellBytes;
    const char *tile0 = w + (size_t)blockIdx.x * CB * tile_bytes;

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));

    floatx4 Y[CB];
#pragma unroll
    for (int c = 0; c < CB; ++c) Y[c] = floatx4{0.f, 0.f, 0.f, 0.f};

    const bool row_valid = ln < M;
    const uint16_t *xrow = x + (size_t)(row_valid ? ln : 0) * K + 8 * lg;
    const int ntasks = (G + kGemmWsGroups - 1) / kGemmWsGroups;
    // The scale words of a task (4 groups x CB tiles x 16 columns: one 16-byte chunk per tile and column, since the
    // task's groups are one aligned quad of a block) are fetched by one request of the wave, lane (c, ln) taking tile
    // c's chunk, and handed to the lanes that need them through a KiB of LDS private to the wave.  Fetched as
    // sixteen 4-byte loads per wave they cost as many address-unit cycles as the task's cells (M = 16, K = 4096,
    // N = 14336: 9.9 -> 9.2 us on cached weights, 10.4 -> 10.3 us cold); as 16-byte loads of every lane they do not
    // fit the 256 registers.
    //
    // Where the time goes at that shape (requests replaced by constants, cold): 3.6 us without any x or cell request,
    // +2.9 us for the x requests alone (128 KB per workgroup, L2 hits), +4.0 us for the cells alone (143 KB per
    // workgroup from HBM), 10.3 us with both: the two streams add up, i.e. a CU takes in ~40 bytes per ns whatever the
    // source.  Not kept, no gain: x copied to LDS once per workgroup with whole-line requests (10.3 - 10.4 us); the 896
    // tiles dealt 4 and 3 to 256 workgroups instead of 4 to 224 (10.55 against 10.59 us on one box).
    // (Q4NX order: one such request and KiB per K-step, lane (c, ln) of KiB t holding the task's four (scale, min) pairs of
    // rows 32 t .. 32 t + 31.)
    u32x4 *mdl = reinterpret_cast<u32x4 *>(red + kGemmWsWaves * CB * 4 * 64) + wave * 64 * MDK;
    for (int task = wave; task < ntasks; task += kGemmWsWaves) {
        const int g0 = task * kGemmWsGroups;
        u32x4 X[kGemmWsGroups][4], cell[kGemmWsGroups][CB];
        u32x4 mdq[MDK];
        {
            const int b = g0 >> 4, gl = g0 & 15, c = lg < CB ? lg : CB - 1;
            const char *src = tile0 + (size_t)c * tile_bytes + (size_t)b * ((kWsBlockGroups + MDK) * kWsCellBytes) + (16 * (gl >> 2) + ln) * 16;
#pragma unroll
            for (int t = 0; t < MDK; ++t) mdq[t] = *reinterpret_cast<const u32x4 *>(src + (size_t)t * kWsCellBytes);
        }
#pragma unroll
        for (int j = 0; j < kGemmWsGroups; ++j) {
            const int g = g0 + j < G ? g0 + j : G - 1;   // a short last task re-reads the last group (its x is zeroed below)
#pragma unroll
            for (int t = 0; t < 4; ++t) X[j][t] = *reinterpret_cast<const u32x4 *>(xrow + 128 * g + 32 * t);
        }
#pragma unroll
        for (int j = 0; j < kGemmWsGroups; ++j) {
            const int g = g0 + j < G ? g0 + j : G - 1;
            const int b = g >> 4, gl = g & 15;
            const char *blk = tile0 + (size_t)b * ((kWsBlockGroups + MDK) * kWsCellBytes);
#pragma unroll
            for (int c = 0; c < CB; ++c)
                cell[j][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(blk + (size_t)c * tile_bytes + (size_t)(MDK + gl) * kWsCellBytes) + lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        // (LDS operations of one wave complete in order; the previous task's reads are done)
#pragma unroll
        for (int t = 0; t < MDK; ++t) mdl[64 * t + lane] = mdq[t];
        if constexpr (Q4) {
            const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < kGemmWsGroups; ++j) {
                const bool valid = row_valid && g0 + j < G;
                floatx4 xs[4];   // xs[t][i]: sum of x[4 lg + i] over rows 32 t .. 32 t + 31 of the group
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (!valid) X[j][t] = u32x4{0u, 0u, 0u, 0u};
                    xs[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][t]), ones, zero4, 0, 0, 0);
                }
#pragma unroll
                for (int c = 0; c < CB; ++c) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const floatx4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][t]),
                                                                                    cell_operand(cell[j][c][t], nib_mask, magic), zero4, 0, 0, 0);
                        // the pair of (group g0 + j, K-step t, column ln) of tile c: dword j of the chunk lane 16 c + ln fetched
                        uint32_t mw = reinterpret_cast<const uint32_t *>(mdl + 64 * t + 16 * c + ln)[j];
                        if (g0 + j >= G) mw = 0u;   // (a short last task: no such group)
                        const float sf = __builtin_bit_cast(float, mw << 16);
                        const float c2 = fmaf(-128.0f, sf, __builtin_bit_cast(float, mw & 0xFFFF0000u));   // min - 128 s
#pragma unroll
                        for (int i = 0; i < 4; ++i) Y[c][i] = fmaf(sf, acc[i], fmaf(c2, xs[t][i], Y[c][i]));
                    }
                }
            }
            continue;
        }
        // the scale word of (group g0 + j, column ln) of tile c: dword j of the chunk that lane 16 c + ln fetched
        u32x4 md[CB];
#pragma unroll
        for (int cc = 0; cc < CB; ++cc) md[cc] = mdl[16 * cc + ln];
#pragma unroll
        for (int j = 0; j < kGemmWsGroups; ++j) {
            const bool valid = row_valid && g0 + j < G;
            floatx4 xs = {0.f, 0.f, 0.f, 0.f};   // register i: sum of x[4 lg + i] over the group
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                if (!valid) X[j][t] = u32x4{0u, 0u, 0u, 0u};
                xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][t]), ones, xs, 0, 0, 0);
            }
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][t]),
                                                                  cell_operand(cell[j][c][t], nib_mask, magic), acc, 0, 0, 0);
                const uint32_t mw = g0 + j < G ? md[c][j] : 0u;   // (a short last task: no such group, s = 0)
                const float sf = __builtin_bit_cast(float, mw << 16);
                const float nz = __builtin_bit_cast(float, mw & 0xFFFF0000u);   // -(128 + z)
#pragma unroll
                for (int i = 0; i < 4; ++i) Y[c][i] = fmaf(sf, fmaf(nz, xs[i], acc[i]), Y[c][i]);
            }
        }
    }

    // cross-wave sum: red[wave][c][i][lane], then every thread adds the waves for two (row, column) pairs
#pragma unroll
    for (int c = 0; c < CB; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((wave * CB + c) * 4 + i) * 64 + lane] = Y[c][i];
    __syncthreads();
    constexpr int PER_WAVE = CB * 4 * 64;
    for (int e = threadIdx.x; e < PER_WAVE; e += kGemmWsWaves * 64) {
        // e = (m * CB + c) * 16 + col: consecutive threads write consecutive columns of one row
        const int col = e & 15, c = (e >> 4) % CB, m = e / (16 * CB);
        const int src = (c * 4 + (m & 3)) * 64 + 16 * (m >> 2) + col;   // row m lives in lane group m / 4, register m % 4
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < kGemmWsWaves; ++wv) s += red[wv * PER_WAVE + src];
        if (m < M) {
            const size_t o = (size_t)m * N + (size_t)blockIdx.x * (16 * CB) + 16 * c + col;
            if (residual) s += bf16_bits_to_float(residual[o]);
            y[o] = float_to_bf16_bits(s);
        }
    }
}

// 17 <= M <= 64 in one launch: RT row tiles of 16.  The same plan as gemm_ws_kernel (a workgroup owns CB tiles for all of
// K, its waves take the tasks round-robin and meet in LDS), with a cell's B operand built once and multiplied with RT A
// operands.  A task is 4 / RT groups (RT = 4: one), so that the x operands of a task stay at 64 registers; the scale
// words are read from the task's KiB one dword at a time, because which dword of a chunk belongs to the task's group
// depends on the group.  AWQ order only.
template <int CB, int RT>
__global__ void __launch_bounds__(kGemmWsWaves * 64) gemm_ws_rows_kernel(const uint16_t *__restrict__ x, const char *__restrict__ w,
                                                                         uint16_t *__restrict__ y, int M, int K, int N, int G, int NB) {
    constexpr int GPT = 4 / RT;   // groups per task
    static_assert(RT == 2 || RT == 4, "row tiles per launch");
    extern __shared__ __attribute__((aligned(16))) float red[];   // [wave][row tile][cb][reg][lane]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lg = lane >> 4, ln = lane & 15;
    const size_t tile_bytes = (size_t)(NB + G) * kWsCellBytes;
    const char *tile0 = w + (size_t)blockIdx.x * CB * tile_bytes;

    const uint32_t ones_w = 0x3F803F80u;
    const u32x4 ones4 = {ones_w, ones_w, ones_w, ones_w};
    const bf16x8 ones = __builtin_bit_cast(bf16x8, ones4);
    uint32_t nib_mask = 0x000F000Fu, magic = 0x43004300u;
    asm volatile("" : "+s"(nib_mask));
    asm volatile("" : "+v"(magic));

    floatx4 Y[RT][CB];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int c = 0; c < CB; ++c) Y[rt][c] = floatx4{0.f, 0.f, 0.f, 0.f};

    bool row_valid[RT];
    const uint16_t *xrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        row_valid[rt] = 16 * rt + ln < M;
        xrow[rt] = x + (size_t)(row_valid[rt] ? 16 * rt + ln : 0) * K + 8 * lg;
    }
    const int ntasks = (G + GPT - 1) / GPT;
    u32x4 *mdl = reinterpret_cast<u32x4 *>(red + kGemmWsWaves * RT * CB * 4 * 64) + wave * 64;
    for (int task = wave; task < ntasks; task += kGemmWsWaves) {
        const int g0 = task * GPT;
        u32x4 X[GPT][RT][4], cell[GPT][CB];
        u32x4 mdq;
        {   // the chunk of the aligned quad of groups that holds the task's: lane (c, ln) takes tile c's
            const int b = g0 >> 4, gl = g0 & 15, c = lg < CB ? lg : CB - 1;
            mdq = *reinterpret_cast<const u32x4 *>(tile0 + (size_t)c * tile_bytes + (size_t)b * ((kWsBlockGroups + 1) * kWsCellBytes) +
                                                   (16 * (gl >> 2) + ln) * 16);
        }
#pragma unroll
        for (int j = 0; j < GPT; ++j) {
            const int g = g0 + j < G ? g0 + j : G - 1;   // a short last task re-reads the last group (its x is zeroed below)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int t = 0; t < 4; ++t) X[j][rt][t] = *reinterpret_cast<const u32x4 *>(xrow[rt] + 128 * g + 32 * t);
        }
#pragma unroll
        for (int j = 0; j < GPT; ++j) {
            const int g = g0 + j < G ? g0 + j : G - 1;
            const int b = g >> 4, gl = g & 15;
            const char *blk = tile0 + (size_t)b * ((kWsBlockGroups + 1) * kWsCellBytes);
#pragma unroll
            for (int c = 0; c < CB; ++c)
                cell[j][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(blk + (size_t)c * tile_bytes + (size_t)(1 + gl) * kWsCellBytes) + lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        mdl[lane] = mdq;   // (LDS operations of one wave complete in order; the previous task's reads are done)
#pragma unroll
        for (int j = 0; j < GPT; ++j) {
            const bool have = g0 + j < G;
            floatx4 xs[RT];   // xs[rt][i]: sum of x[16 rt + 4 lg + i] over the group
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                xs[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (!(row_valid[rt] && have)) X[j][rt][t] = u32x4{0u, 0u, 0u, 0u};
                    xs[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][rt][t]), ones, xs[rt], 0, 0, 0);
                }
            }
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                floatx4 acc[RT];
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const bf16x8 bop = cell_operand(cell[j][c][t], nib_mask, magic);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, X[j][rt][t]), bop, acc[rt], 0, 0, 0);
                }
                // the scale word of (group g0 + j, column ln) of tile c: dword (g0 + j) % 4 of the chunk lane 16 c + ln fetched
                uint32_t mw = reinterpret_cast<const uint32_t *>(mdl + 16 * c + ln)[(g0 + j) & 3];
                if (!have) mw = 0u;   // (a short last task: no such group, s = 0)
                const float sf = __builtin_bit_cast(float, mw << 16);
                const float nz = __builtin_bit_cast(float, mw & 0xFFFF0000u);   // -(128 + z)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) Y[rt][c][i] = fmaf(sf, fmaf(nz, xs[rt][i], acc[rt][i]), Y[rt][c][i]);
            }
        }
    }

    // cross-wave sum: red[wave][rt][c][i][lane], then every thread adds the waves for its (row, column) pairs
    constexpr int PER_TILE = CB * 4 * 64, PER_WAVE = RT * PER_TILE;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave * PER_WAVE + rt * PER_TILE + (c * 4 + i) * 64 + lane] = Y[rt][c][i];
    __syncthreads();
    for (int e = threadIdx.x; e < PER_WAVE; e += kGemmWsWaves * 64) {
        // e = (m * CB + c) * 16 + col: consecutive threads write consecutive columns of one row
        const int col = e & 15, c = (e >> 4) % CB, m = e / (16 * CB);
        const int mt = m & 15;   // row m lives in row tile m / 16, lane group mt / 4, register mt % 4
        const int src = (m >> 4) * PER_TILE + (c * 4 + (mt & 3)) * 64 + 16 * (mt >> 2) + col;
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < kGemmWsWaves; ++wv) s += red[wv * PER_WAVE + src];
        if (m < M) y[(size_t)m * N + (size_t)blockIdx.x * (16 * CB) + 16 * c + col] = float_to_bf16_bits(s);
    }
}

template <int CB, int RT>
hipError_t launch_gemm_ws_rows(const uint16_t *x, const void *w, uint16_t *y, int M, int K, int N, hipStream_t stream) {
    const size_t lds = (size_t)kGemmWsWaves * RT * CB * 4 * 64 * sizeof(float) + kGemmWsWaves * kWsCellBytes;   // sums, scale words
    if (lds >= 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_ws_rows_kernel<CB, RT>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemm_ws_rows_kernel<CB, RT>), dim3(N / (16 * CB)), dim3(kGemmWsWaves * 64), lds, stream, x,
                       static_cast<const char *>(w), y, M, K, N, K / kGroup, ws_blocks(K));
    return hipGetLastError();
}

template <int CB, bool Q4>
hipError_t launch_gemm_ws_q(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, int M, int K, int N,
                            hipStream_t stream) {
    const size_t lds = (size_t)kGemmWsWaves * CB * 4 * 64 * sizeof(float) + kGemmWsWaves * kWsCellBytes * (Q4 ? kWsQ4MdKiB : 1);   // sums, scale words
    if (lds >= 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_ws_kernel<CB, Q4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((gemm_ws_kernel<CB, Q4>), dim3(N / (16 * CB)), dim3(kGemmWsWaves * 64), lds, stream, x,
                       static_cast<const char *>(w), y, residual, M, K, N, K / kGroup, ws_blocks(K));
    return hipGetLastError();
}

template <int CB>
hipError_t launch_gemm_ws_cb(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, int M, int K, int N,
                             hipStream_t stream, bool q4) {
    return q4 ? launch_gemm_ws_q<CB, true>(x, w, y, residual, M, K, N, stream) : launch_gemm_ws_q<CB, false>(x, w, y, residual, M, K, N, stream);
}

}  // namespace

// y[M, N] = bf16(x[M, K] . W (+ residual)): up to 64 rows per launch (Q4NX order, or with a residual: 16), more rows as
// further launches.
hipError_t launch_gemm_ws(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, int M, int K, int N,
                          hipStream_t stream, bool q4) {
    const int tiles = N / kWsTileCols;
    int cb = g_gemv_ws_tune.cb;
    if (!cb) cb = tiles % 4 == 0 && tiles / 4 >= 200 ? 4 : (tiles % 2 == 0 && tiles / 2 >= 200 ? 2 : 1);
    if (tiles % cb) cb = 1;
    hipError_t e = hipSuccess;
    // (the launches of several row tiles take the AWQ order and no residual)
    const int max_rows = q4 || residual || g_gemv_ws_tune.gemm_rows == 16 ? 16 : (g_gemv_ws_tune.gemm_rows == 32 ? 32 : 64);
    for (int m0 = 0; m0 < M && e == hipSuccess;) {
        const int rows = M - m0 < max_rows ? M - m0 : max_rows;
        const uint16_t *xr = x + (size_t)m0 * K, *rr = residual ? residual + (size_t)m0 * N : nullptr;
        uint16_t *yr = y + (size_t)m0 * N;
        if (rows > 32)
            e = cb == 4 ? launch_gemm_ws_rows<4, 4>(xr, w, yr, rows, K, N, stream)
              : cb == 2 ? launch_gemm_ws_rows<2, 4>(xr, w, yr, rows, K, N, stream)
                        : launch_gemm_ws_rows<1, 4>(xr, w, yr, rows, K, N, stream);
        else if (rows > 16)
            e = cb == 4 ? launch_gemm_ws_rows<4, 2>(xr, w, yr, rows, K, N, stream)
              : cb == 2 ? launch_gemm_ws_rows<2, 2>(xr, w, yr, rows, K, N, stream)
                        : launch_gemm_ws_rows<1, 2>(xr, w, yr, rows, K, N, stream);
        else
            e = cb == 4 ? launch_gemm_ws_cb<4>(xr, w, yr, rr, rows, K, N, stream, q4)
              : cb == 2 ? launch_gemm_ws_cb<2>(xr, w, yr, rr, rows, K, N, stream, q4)
                        : launch_gemm_ws_cb<1>(xr, w, yr, rr, rows, K, N, stream, q4);
        m0 += rows;
    }
    return e;
}

}  // namespace w4a16
