// Internal launch interface between the C ABI (capi.hip) and the kernel files.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace w4a16 {

// Layout of the caller-provided workspace: [kHeaderBytes header: word 0 counts poll
// timeouts][fp32 split-K partial slots].  Between calls every slot holds 0xFFFFFFFF.
constexpr size_t kHeaderBytes = 256;
constexpr int kMaxKSplit = 32;
constexpr int kStreamMaxM = 96;   // up to here w4a16_gemm_bf16 runs the streaming kernel in 16-row launches
constexpr int kGemmWsMaxM = 128;  // up to here w4a16_gemm_stream_bf16 runs the batched kernel (launches of up to 64 rows)

struct StreamTune {
    int lw = 0;       // packed words per lane per row: 1, 2 or 4 (tile = 128 * lw columns)
    int ksteps = 0;   // K-steps (32 rows) a wave loads per unit: 1, 2 or 4 (0 = heuristic)
    int waves = 0;    // waves per workgroup: 4 or 8
    int units = 0;    // units each wave processes back to back
    int ksplit = 0;   // workgroups along K per tile (overrides units)
    int stream_max_m = 0;   // largest M that w4a16_gemm_bf16 gives to the streaming kernel (0 = kStreamMaxM; at least 16)
    int skip_publish = 0; // tests only: producers do not publish, so reducers run into their poll bound
    int spin_limit = 0;   // reducer poll bound (0 = default); tiny values force the timeout path in tests
    int no_attn_fuse = 0; // 1: w4a16_decode_attn_o_gemv_ffn_bf16 always runs the attention merge launch
};
extern StreamTune g_stream_tune;

struct StreamPlan {
    int lw, ksteps, waves, units, ksplit, ntiles, mi;
};
StreamPlan plan_stream(int M, int K, int N, bool fixed_shape = false);   // fixed_shape: 256-column tiles, 8 waves, whatever the tune keys say

hipError_t launch_dequant(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, uint16_t *out,
                          int K, int N, hipStream_t stream);

// 1-D dequant of the reference's tiled [herd_n, tile_bytes] buffer (dequant.hip).
hipError_t launch_dequant_1d(const uint8_t *packed, uint16_t *out, int n, int gs, int herd_n, hipStream_t stream);

// Optional stages fused into the streaming kernel.
struct StreamExtras {
    const uint16_t *residual = nullptr;   // [M, N] bf16 added to the result before the final rounding
    int round_before_add = 0;             // 1: y = bf16(bf16(x.W) + R) instead of bf16(x.W + R)
    const uint16_t *norm_w = nullptr;     // [K] bf16: x is replaced by bf16((x * rstd) * norm_w), M <= 4
    float eps = 1e-5f;
    // M == 1 only.  A launch with `sumsq_out` leaves the sum of squares of its (rounded) outputs there,
    // one float per 256-column tile; a following RMS launch on that vector passes it as `sumsq_in`
    // (`sumsq_n` <= 64 pieces) and skips reading x for the norm.
    const float *sumsq_in = nullptr;
    int sumsq_n = 0;
    float *sumsq_out = nullptr;
    // M == 1: x is not read; it is the merge of the decode attention's per-chunk partials (attention_partials below),
    // computed by every wave for the rows of its units exactly as the attention merge kernel computes it.  Only where
    // stream_attn_fusable says so.
    const float *attn_ml = nullptr;    // [n_heads, nsplit, 2]
    const float *attn_acc = nullptr;   // [n_heads, nsplit, head_dim]
    int attn_nsplit = 0, attn_hd = 0;
};
bool stream_attn_fusable(int K, int N, int head_dim, int nsplit);

// y[M, N] = bf16(x[M, K] . W), M <= 16.  With `up_*` given (SwiGLU epilogue, M == 1) the
// kernel streams both weight sets and writes y = bf16(silu(bf16(x.Wg)) * bf16(x.Wu)).
hipError_t launch_stream(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                         const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                         uint16_t *y, int M, int K, int N, void *workspace, hipStream_t stream,
                         const StreamExtras &extras = StreamExtras());

// Prefill GEMM (M > 16) with an optional epilogue on a second bf16 [M, N] operand `aux`:
//   kEpiAddRounded   y = bf16(bf16(x . W) + aux)            (residual add of a bf16 product)
//   kEpiSiluGateMul  y = bf16(silu(aux) * bf16(x . W))      (SwiGLU with aux = the gate projection)
//   kEpiRope         half-split RoPE of the bf16 product on columns [0, rope.cols) (whole heads of rope.head_dim,
//                    64 or 128), aux = the LUT [positions, head_dim] (cos then sin), row m at position rope.pos0 + m
enum : int { kEpiNone = 0, kEpiAddRounded = 1, kEpiSiluGateMul = 2, kEpiRope = 3 };
struct GemmRope {
    int cols, head_dim, pos0;
};
// With `splitk_scratch` (plain scratch of gemm_prefill_splitk_bytes) a launch with few tiles is cut into 2 or 4
// slices along K whose fp32 partial products a second kernel sums before the epilogue.
hipError_t launch_gemm_prefill(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                               const uint16_t *scales, uint16_t *y, int M, int K, int N, hipStream_t stream,
                               int epi = kEpiNone, const uint16_t *aux = nullptr, float *splitk_scratch = nullptr,
                               int cus = 0, const GemmRope *rope = nullptr);
int gemm_prefill_ksplit(int M, int K, int N, int cus);
size_t gemm_prefill_splitk_bytes(int M, int K, int N, int cus);

hipError_t launch_fill_workspace(void *ptr, size_t bytes, hipStream_t stream);

// Whole-K decode GEMV on the stream-order layout (gemv_ws.hip, layout in wstream.h): stateless, no workspace.
struct GemvWsExtras {
    const uint16_t *residual = nullptr;   // [N] bf16 added to the result before the final rounding
    int round_before_add = 0;             // 1: y = bf16(bf16(x.W) + R) instead of bf16(x.W + R)
    const uint16_t *norm_w = nullptr;     // [K] bf16: x is replaced by bf16((x * rstd) * norm_w)
    float eps = 1e-5f;
    // A launch with `sumsq_out` leaves the sum of squares of its (rounded) outputs there, one float per
    // 16-column tile (N / 16 floats); a following RMS launch on that vector passes them as `sumsq_in`
    // (`sumsq_n` pieces) and skips its own pass over x.
    const float *sumsq_in = nullptr;
    int sumsq_n = 0;
    float *sumsq_out = nullptr;
    bool q4 = false;                      // the matrices are in Q4NX order (a scale and a min per 32 rows)
};
struct GemvWsTune {
    int ct = 0;      // cells (groups) per task: 4, 8 or 16 (0 = default)
    int waves = 0;   // cap on the waves per workgroup (0 = one per task, at most 16)
    int cb = 0;      // batched kernel: 16-column tiles per workgroup, 1, 2 or 4 (0 = by the number of tiles)
    int prefill_tile = 0;    // prefill kernel: 0 = by shape, 1 = 128 x 448 tiles, 2 = 256 x 256 tiles
    int gemm_rows = 0;       // batched kernel: most rows per launch, 16, 32 or 64 (0 = 64)
    int prefill_min_m = 0;   // smallest M that w4a16_gemm_stream_bf16 gives to the prefill kernel (0 = default)
    int prefill_band = 0;    // prefill kernel: row panels per band of the tile order (0 = default)
    int splitk = 0;          // w4a16_gemm_stream_scratch_bf16 at 17 .. 128 rows: 0 split-K where it pays by shape, 1 always, 2 never
    int prefill_swiglu_split = 0;   // 1: the prompt-pass FFN runs gate and up as two launches instead of one
};
extern GemvWsTune g_gemv_ws_tune;
struct GemvWsPlan {
    int ct, waves;
};
GemvWsPlan plan_gemv_ws(int K, int nmat, int N, bool rms);
// y[N] = bf16(x[K] . W) with W in stream order; with `w_up` (second matrix, same shape) the SwiGLU epilogue
// y = bf16(silu(bf16(x.W)) * bf16(x.W_up)).
hipError_t launch_gemv_ws(const uint16_t *x, const void *w, const void *w_up, uint16_t *y, int K, int N, hipStream_t stream,
                          const GemvWsExtras &extras = GemvWsExtras());
// Read-only pass over a stream-order matrix in the GEMV's launch shape; `out` takes one word per wave (N / 16 * 16 words).
hipError_t launch_probe_ws(const void *w, uint32_t *out, int K, int N, hipStream_t stream);
// y[M, N] = bf16(x[M, K] . W (+ residual [M, N])) with W in stream order, any M >= 2 (launches of up to 64 rows; Q4NX order: 16).
hipError_t launch_gemm_ws(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, int M, int K, int N,
                          hipStream_t stream, bool q4 = false);   // q4: W in Q4NX order
// Batched decode split along K (gemm_wsk.hip), 17 <= M: launches of up to 64 rows, each followed by the launch that adds the
// slices; `scratch`: gemm_wsk_scratch_bytes(M, K, N) bytes of plain scratch (0: not needed, one slice).
size_t gemm_wsk_scratch_bytes(int M, int K, int N);
bool gemm_wsk_pays(int M, int K, int N);   // the split is the faster of the two for this shape (or forced by the tune key)
hipError_t launch_gemm_wsk(const uint16_t *x, const void *w, uint16_t *y, const uint16_t *residual, float *scratch, int M, int K,
                           int N, hipStream_t stream);
// Prefill GEMM on stream-order weights (gemm_ws.hip): bf16-rounded weights dequantised in registers, x through LDS.
bool gemm_prefill_ws_supported(int M, int K, int N);   // K % 256 == 0, N % 64 == 0
// Epilogues as for launch_gemm_prefill (kEpi*); kEpiRope with heads of 128 needs N % 128 == 0.
// `q4`: the matrix is in Q4NX order (launch_repack_ws_q4), W = bf16_rne(q s + min').
hipError_t launch_gemm_prefill_ws(const uint16_t *x, const void *w, uint16_t *y, int M, int K, int N, hipStream_t stream,
                                  int epi = kEpiNone, const uint16_t *aux = nullptr, const GemmRope *rope = nullptr, bool q4 = false);
// h[M, H] = bf16(silu(bf16(x . W_gate)) * bf16(x . W_up)) in one launch (H % 64 == 0): bit for bit the gate launch followed
// by the up launch with kEpiSiluGateMul.
hipError_t launch_gemm_prefill_ws_swiglu(const uint16_t *x, const void *w_gate, const void *w_up, uint16_t *h, int M, int K, int H,
                                         hipStream_t stream, bool q4 = false);
// Operands of the affine path (q4nx_repack: qweight [K, N / 8], scales and mins [K / 32, N]) -> Q4NX order
// (ws_q4_matrix_bytes(K, N) bytes at `out`).
hipError_t launch_repack_ws_q4(const int32_t *qweight, const uint16_t *scales, const uint16_t *mins, void *out, int K, int N,
                               hipStream_t stream);
// AutoAWQ checkpoint tensors -> stream order (ws_matrix_bytes(K, N) bytes at `out`).
hipError_t launch_repack_ws(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, void *out, int K, int N,
                            hipStream_t stream);

// Prefill O projection + FFN block (prefill_block.hip): five launches, intermediates in the workspace
// (plain scratch, no initialisation).
struct PrefillLinear {
    const int32_t *qw, *qz;
    const uint16_t *sc;
};
bool prefill_block_supported(int M, int E, int H);
size_t prefill_block_scratch_bytes(int M, int E, int H);   // sized for split-K on a 256-CU device
hipError_t launch_rmsnorm_rows(const uint16_t *x, const uint16_t *w, uint16_t *out, int M, int K, float eps, hipStream_t stream);
// Causal GQA attention over the M rows of a prefill (prefill_attention.hip); qkv is [M, (n_heads + 2 n_kv) * head_dim].
hipError_t launch_prefill_attention(const uint16_t *qkv, uint16_t *attn_out, int M, int n_heads, int n_kv, int head_dim,
                                    hipStream_t stream);
// RMSNorm rows + fused Q|K|V GEMM + RoPE on the Q and K heads (prefill_block.hip); `normed` [M, E] is scratch.
hipError_t launch_prefill_rms_qkv_rope(const uint16_t *x, const uint16_t *norm_w, float eps, const PrefillLinear &wqkv,
                                       const uint16_t *rope_lut, int pos0, uint16_t *qkv_out, int M, int E, int n_heads,
                                       int n_kv, int head_dim, uint16_t *normed, hipStream_t stream);
hipError_t launch_prefill_o_ffn(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_w, float eps,
                                const PrefillLinear &wo, const PrefillLinear &wg, const PrefillLinear &wu,
                                const PrefillLinear &wd, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                int H, void *workspace, int cus, hipStream_t stream);
// The same blocks on stream-order weights (every matrix re-packed with launch_repack_ws; `q4`: with launch_repack_ws_q4).
bool prefill_block_stream_supported(int M, int E, int H);
hipError_t launch_prefill_rms_qkv_rope_stream(const uint16_t *x, const uint16_t *norm_w, float eps, const void *wqkv,
                                              const uint16_t *rope_lut, int pos0, uint16_t *qkv_out, int M, int E, int n_heads,
                                              int n_kv, int head_dim, uint16_t *normed, hipStream_t stream, bool q4 = false);
hipError_t launch_prefill_o_ffn_stream(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_w, float eps,
                                       const void *wo, const void *wg, const void *wu, const void *wd, uint16_t *y,
                                       uint16_t *res1_out, uint16_t *h_out, int M, int E, int H, void *workspace,
                                       hipStream_t stream, bool q4 = false);

// Q4NX / Q4_0 block codec (q4nx.hip).  mode: 0 w = s q + m, 1 w = s (q - m), 2 signed q, w = s q.
hipError_t launch_q4nx_dequant(const void *blocks, uint16_t *out, int M, int K, int mode, hipStream_t stream);
hipError_t launch_q4nx_repack(const void *blocks, int32_t *qweight, uint16_t *scales, uint16_t *mins, int M, int K,
                              int mode, hipStream_t stream);
// Blocks of W[M, K] -> Q4NX stream order of the [K, N = M] matrix (ws_q4_matrix_bytes(K, M) bytes) in one pass.
hipError_t launch_q4nx_blocks_to_stream(const void *blocks, void *out, int M, int K, int mode, hipStream_t stream);

// Final RMSNorm + bf16 lm_head GEMV + argmax (lm_head.hip).  The scratch buffer holds one 8-byte
// argmax key per 16 rows and needs no initialisation.
bool lm_head_supported(int V, int E);
size_t lm_head_scratch_bytes(int V);
hipError_t launch_lm_head(const uint16_t *x, const uint16_t *norm_w, float eps, const uint16_t *w, uint16_t *logits,
                          int32_t *argmax_out, int V, int E, void *workspace, hipStream_t stream);

// Decode attention (attention.hip).  The scratch buffer holds per-chunk softmax partials and
// needs no initialisation.
constexpr int kMaxAttnSplit = 32;
int attention_nsplit(int seq_len);
size_t attention_workspace_bytes(int n_heads, int head_dim);
hipError_t launch_decode_attention(const uint16_t *qkv, const uint16_t *lut_row, uint16_t *k_cache, uint16_t *v_cache,
                                   uint16_t *out, int pos, int max_seq, int n_heads, int n_kv, int head_dim,
                                   void *workspace, hipStream_t stream, bool combine = true);
// Where launch_decode_attention(..., combine = false) leaves its partials inside the attention scratch buffer.
inline void attention_partials(void *workspace, int n_heads, const float **ml, const float **acc) {
    *ml = reinterpret_cast<const float *>(workspace);
    *acc = *ml + (size_t)n_heads * kMaxAttnSplit * 2;
}

// Half-split RoPE of rows x dim bf16 with one LUT row (cos then sin) per row (attention.hip).
hipError_t launch_rope_rows(const uint16_t *x, const uint16_t *lut, uint16_t *out, int rows, int dim, hipStream_t stream);

}  // namespace w4a16
