/*
 * w4a16.h - C ABI of the MI355X (gfx950) AWQ int4 / W4A16 kernels.
 *
 * One shared library (libw4a16_hip.so).  All data pointers are DEVICE pointers owned by
 * the caller; nothing here allocates or frees device memory.  Every entry point returns
 * W4A16_OK (0) or a negative W4A16_ERR_* code.  Arguments are validated before the first
 * HIP call, so every error path below can be exercised on a host without a GPU.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream); launches are
 * asynchronous on that stream.
 *
 * Tensor conventions (AutoAWQ "gemm" layout, the reference's checkpoint format,
 * programming_examples/llms/llama32_1b_int4/awq_repacker.py:7-11):
 *   qweight  int32 [K, N/8]   8 uint4 per word along N; bit position 4*i holds column
 *                             8*b + {0,2,4,6,1,3,5,7}[i]      (awq_repacker.py:33-38)
 *   qzeros   int32 [K/group, N/8]  same packing
 *   scales   bf16  [K/group, N]    (uint16 bit patterns)
 *   x        bf16  [M, K] row-major,  y  bf16 [M, N] row-major,  y = x . W
 *   W[k, n] = (q[k, n] - z[k/group, n]) * s[k/group, n]
 * The examples' D[out] = A[out, K] @ B[K] (matvec_int4_packed.py:4) is the same product
 * with out = N.
 *
 * Constraints: group == 128, K % 128 == 0, N % 8 == 0 for the dequant and N % 32 == 0
 * for GEMV / GEMM / FFN, 16-byte aligned pointers.
 */
#ifndef W4A16_H
#define W4A16_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define W4A16_OK 0
#define W4A16_ERR_NULL (-1)        /* a required pointer is NULL */
#define W4A16_ERR_SHAPE (-2)       /* M/K/N non-positive or not a supported multiple */
#define W4A16_ERR_GROUP (-3)       /* group size other than 128 */
#define W4A16_ERR_ALIGN (-4)       /* a pointer is not 16-byte aligned */
#define W4A16_ERR_WORKSPACE (-5)   /* workspace missing or smaller than *_workspace_bytes */
#define W4A16_ERR_HIP (-6)         /* a HIP call failed; see w4a16_last_hip_error() */
#define W4A16_ERR_TUNE (-7)        /* unknown tuning key or value out of range */
#define W4A16_ERR_TIMEOUT (-8)     /* w4a16_workspace_check: a split-K reducer timed out */
#define W4A16_ERR_TOO_LARGE (-9)   /* w4a16_gemv_noalloc_bf16: shape beyond its fixed scratch */
#define W4A16_ERR_NOT_PREPARED (-10) /* w4a16_gemv_noalloc_bf16: first use on this GPU under stream capture */

#define W4A16_ABI_VERSION 1

int w4a16_abi_version(void);

/* Static description of an error code (never NULL). */
const char *w4a16_strerror(int code);

/* hipGetErrorString of the last failing HIP call on this thread ("" if none). */
const char *w4a16_last_hip_error(void);

/*
 * Dense dequant: out[k, n] = bf16_rne((q - z) * s), bit-exact with the reference's
 * awq_dequant_layer (programming_examples/llms/llama32_1b_int4/awq_pack.py:84-104) and
 * dequant_to_bf16 (awq_repacker.py:57-82).  Replaces the device kernel
 * dequant_int4_bf16(uint8_t *packed, bfloat16 *out)
 * (programming_examples/dequant_awq/dequant.cc:77-85).
 */
int awq_dequant_bf16(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                     uint16_t *out_bf16, int K, int N, int group, void *stream);

/*
 * 1-D dequant on the reference example's own packed buffer: out[i] = bf16_rne((q[i] - z[i / group]) * s[i / group]),
 * i < n.  `packed` is uint8 [herd_n, tile_bytes] as pack_inputs builds it
 * (programming_examples/dequant_awq/dequant_awq.py:259-278): per tile of n / herd_n elements
 * [Q: two elements per byte, the even one in the low nibble][S: bf16 per group][Z: u8 per group], padded to a
 * multiple of 4 bytes (packed_tile_bytes, dequant_awq.py:59-69); awq_dequant_1d_tile_bytes returns that size (0 for
 * an unsupported shape).  Same entry as the device kernel dequant_int4_bf16(uint8_t *packed, bfloat16 *out)
 * (programming_examples/dequant_awq/dequant.cc:77-85), which sees one tile; here one launch covers all tiles.
 * Any group size that is a multiple of 8 with (n / herd_n) % group == 0.
 */
size_t awq_dequant_1d_tile_bytes(int n, int group, int herd_n);
int awq_dequant_1d_bf16(const uint8_t *packed, uint16_t *out_bf16, int n, int group, int herd_n, void *stream);

/*
 * Workspace for the split-K GEMV / small-M GEMM and the FFN.  The caller allocates
 * `*_workspace_bytes` bytes of device memory once, prepares it once with
 * w4a16_workspace_init, and may then reuse it for any number of calls that do not
 * overlap in time (each call leaves it prepared again).  Calls that run concurrently
 * (different streams) need separate workspaces.  The FFN and block entry points keep plain
 * intermediates (h, res1) behind the prepared area, at an offset that depends on their shapes: share
 * a workspace only between calls of one entry point with the same shapes, or prepare it again
 * before a call of another kind.
 */
size_t w4a16_gemm_workspace_bytes(int M, int K, int N);
size_t w4a16_ffn_workspace_bytes(int K, int H);
int w4a16_workspace_init(void *workspace, size_t workspace_bytes, void *stream);

/*
 * Health check (synchronises `stream`): W4A16_ERR_TIMEOUT if any split-K reducer of an
 * earlier call on this workspace gave up waiting for a partial result (its bounded poll ran
 * out; that call's output is invalid and the workspace must be re-initialised), else W4A16_OK.
 */
int w4a16_workspace_check(const void *workspace, void *stream);

/*
 * Decode GEMV, M = 1: y[N] = bf16(x[K] . W).  fp32 accumulation, one bf16 rounding.
 * Replaces matvec_int4_bf16_packed(uint8_t *packed, bfloat16 *b, bfloat16 *c)
 * (programming_examples/matrix_vector_multiplication/int4_awq/mv_int4_bf16.cc:403-411)
 * and matches matvec_int4_packed.cpu_reference (matvec_int4_packed.py:272-287).
 */
int w4a16_gemv_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                    const uint16_t *scales, uint16_t *y, int K, int N, int group,
                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * w4a16_gemv_bf16 without a workspace argument and without any allocation: no counterpart in the
 * reference; it is for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  The split-K partial slots live in a 4.06 MiB
 * device array inside the library (one copy per GPU, held until the process ends), so N <= 32768
 * (W4A16_ERR_TOO_LARGE beyond); other constraints, kernels and results are those of w4a16_gemv_bf16,
 * bit for bit.  The first use on a GPU prepares the array (a fill kernel on `stream`, waited for before
 * anything else may see the array), which a capturing stream cannot do: a first use under stream capture
 * returns W4A16_ERR_NOT_PREPARED and launches nothing; call w4a16_noalloc_check once per GPU outside
 * capture beforehand.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race, exactly as two calls sharing one workspace would.
 *
 * w4a16_noalloc_check(stream) is w4a16_workspace_check for that array (it synchronises `stream`, so not
 * under capture): it prepares the array if this GPU has not used it yet, returns W4A16_ERR_TIMEOUT if a
 * reducer of an earlier w4a16_gemv_noalloc_bf16 call gave up waiting (that call's output is invalid) and
 * then empties the array again, so that the next call is sound; W4A16_OK otherwise.  Allocates nothing.
 */
int w4a16_gemv_noalloc_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                            const uint16_t *scales, uint16_t *y, int K, int N, int group, void *stream);
int w4a16_noalloc_check(void *stream);

/*
 * GEMM, any M >= 1: y[M, N] = bf16(x[M, K] . W).  M <= 16 streams the weights once
 * through a split-K MFMA kernel; M <= 96 does the same in launches of 16 rows (the weights
 * stay cache-resident between them); larger M uses the tiled prefill kernel that dequantises
 * weight tiles to bf16 in LDS (and therefore multiplies bf16-rounded weights).  Replaces matmul_int4_bf16_packed_f32 + f32_to_bf16_mn
 * (mv_int4_bf16.cc:430-448) and matches matmul_int4_packed.cpu_reference
 * (programming_examples/matrix_multiplication/int4_awq/matmul_int4_packed.py:89-105).
 */
int w4a16_gemm_bf16(const uint16_t *x, const int32_t *qweight, const int32_t *qzeros,
                    const uint16_t *scales, uint16_t *y, int M, int K, int N, int group,
                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * Decode FFN front half, batch 1: h[H] = bf16(silu(bf16(x . Wg)) * bf16(x . Wu)), both weight
 * matrices streamed by one kernel.  Matches matvec_int4_swiglu_rms.cpu_reference
 * (programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:501-516) without the
 * RMSNorm prologue; the reference's interleaved gate/up rows are passed as two matrices.
 * Workspace: w4a16_ffn_workspace_bytes(K, H).
 */
int w4a16_gemv_swiglu_bf16(const uint16_t *x,
                           const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                           const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                           uint16_t *h, int K, int H, int group,
                           void *workspace, size_t workspace_bytes, void *stream);

/*
 * Fused decode SwiGLU FFN, batch 1:
 *   g = bf16(x . Wg), u = bf16(x . Wu), h = bf16(silu(g) * u), y = bf16(h . Wd)
 * with silu(g) = g * 0.5 * (tanh(g / 2) + 1) in fp32; Wg, Wu are [K, H], Wd is [H, K].
 * Rounding points follow matvec_int4_swiglu_rms.cpu_reference
 * (programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:512-516) and
 * ld_cpu_reference (programming_examples/llms/llama32_1b_int4/multi_launch_builder/
 * o_gemv_ffn_int4_fused.py:1078-1094) with R = 0 and no RMSNorm prologue.
 * `h_out` (bf16 [H]) may be NULL; when given it receives the intermediate.
 */
int w4a16_ffn_swiglu_bf16(const uint16_t *x,
                          const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                          const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                          const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                          uint16_t *y, uint16_t *h_out, int K, int H, int group,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * Decode GEMV with residual, batch 1: y[N] = bf16(x . W + R), the residual joining the fp32
 * sum before the single rounding.  Replaces matvec_int4_packed_add.cpu_reference
 * (programming_examples/matrix_vector_multiplication/int4_awq/matvec_int4_packed_add.py:302-319)
 * and its device kernel matvec_int4_bf16_packed_add.  `residual` is bf16 [N]; y may alias it.
 * Workspace: w4a16_gemm_workspace_bytes(1, K, N).
 */
int w4a16_gemv_add_bf16(const uint16_t *x,
                        const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                        const uint16_t *residual, uint16_t *y, int K, int N, int group,
                        void *workspace, size_t workspace_bytes, void *stream);

/*
 * Stream order: the device layout of one AWQ matrix for the decode kernels, written once at load
 * time from the checkpoint tensors.  Counterpart of the reference's load-time re-pack of every
 * Linear into the order its cores consume it (repack_for_gemv,
 * programming_examples/llms/llama32_1b_int4/awq_repacker.py:112-135; pack_inputs,
 * programming_examples/matrix_vector_multiplication/int4_awq/matvec_int4_packed.py:57-103).
 * Layout: 16-column tiles, each one contiguous slab holding all K rows as 1 KiB cells of
 * 16 columns x 128 rows (one 128-bit load per lane of a wavefront) with the group's scales and zero
 * points beside them; mlir-air_amd/csrc/wstream.h states it byte by byte.
 * w4a16_stream_bytes(K, N) is the size of the buffer (0 for an unsupported shape); K % 128 == 0,
 * N % 16 == 0, group == 128.
 */
size_t w4a16_stream_bytes(int K, int N);
int w4a16_repack_stream(const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                        void *wstream, int K, int N, int group, void *stream);

/*
 * Decode GEMV on a stream-order matrix, batch 1: y[N] = bf16(x[K] . W), fp32 accumulation, one bf16
 * rounding.  Stateless: a workgroup owns whole columns, so there is no workspace and no exchange
 * between workgroups.  Same reference as w4a16_gemv_bf16: matvec_int4_bf16_packed
 * (programming_examples/matrix_vector_multiplication/int4_awq/mv_int4_bf16.cc:403-411),
 * matvec_int4_packed.cpu_reference (matvec_int4_packed.py:272-287).
 * _add: y = bf16(x . W + R), R bf16 [N] (matvec_int4_packed_add.cpu_reference,
 * matvec_int4_packed_add.py:302-319); y may alias R.
 * _swiglu: h[H] = bf16(silu(bf16(x . Wg)) * bf16(x . Wu)), both matrices [K, H] in stream order
 * (matvec_int4_swiglu_rms.cpu_reference, programming_examples/decode_ffn_swiglu/
 * matvec_int4_swiglu_rms.py:501-516, without the RMSNorm prologue).
 */
int w4a16_gemv_stream_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int K, int N, int group,
                           void *stream);
int w4a16_gemv_add_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual,
                               uint16_t *y, int K, int N, int group, void *stream);
/* Measurement aid, no counterpart among the reference's kernels (its harness times the kernel alone,
 * programming_examples/matrix_vector_multiplication/int4_awq/test_packed.cpp:114-150): one read-only pass over a
 * stream-order matrix with w4a16_gemv_stream_bf16's launch shape and request pattern, everything loaded folded with XOR
 * into out_words (N words: 16 per 16-column tile, one per wave; the others are not written).  Its time is the floor of
 * any kernel that reads the matrix once in that order, which bench.py reports beside the GEMV. */
int w4a16_probe_stream_read(const void *wstream, uint32_t *out_words, int K, int N, void *stream);
/* Batched decode on a stream-order matrix: y[M, N] = bf16(x[M, K] . W), unrounded weights, fp32 accumulation
 * (matmul_int4_packed.cpu_reference, programming_examples/matrix_multiplication/int4_awq/matmul_int4_packed.py:89-105;
 * device kernel matmul_int4_bf16_packed_f32, mv_int4_bf16.cc:430-448).  Up to 64 rows per launch stream the weights
 * once (M <= 128: launches of 64 rows and a rest, the second over cache-resident weights); stateless like the GEMV.  From
 * M = 129 on,
 * with K % 256 == 0 and N % 64 == 0 (N / 64 = 3, 4 or >= 6), the tiled prefill kernel runs instead: it dequantises the
 * weights to bf16 in registers (W = bf16_rne((q - z) * s), the dense dequant's values) and feeds bf16 MFMA with fp32
 * accumulation; other shapes stay with the launches of 64 rows.  So the numerics change between M = 128 and M = 129:
 * below, y is one rounding of the fp32 sum over exact weights (q - z) s, as the reference's cpu_reference computes it;
 * above, the weights carry one more bf16 rounding each (relative 2^-9), which moves y by at most 2^-9 sum |x w| and
 * stays inside the reference's gate (rtol 0.1, atol 0.05, 0.05 % budget, r >= 0.999); a caller that needs the same
 * bits for every M keeps M <= 128 per call.  K % 128 == 0, N % 16 == 0. */
int w4a16_gemm_stream_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int M, int K, int N, int group,
                           void *stream);
/* w4a16_gemm_stream_bf16 with plain scratch for the shapes where 17 .. 128 rows run faster split along K (same
 * reference, matmul_int4_packed.py:89-105; the reference's own kernel also walks K in slices, one L1 K-chunk at a
 * time, and adds them in an fp32 accumulator, matmul_int4_packed.py:179-181, 293-345).  A workgroup takes 256 columns and a slice of K, shares
 * the x rows of its slice through LDS and writes fp32 partial sums to `scratch`; a second launch adds the slices in
 * slice order and rounds once.  That pays where the whole-K launches re-read the x rows most: K >= 4096, rows * K / 128
 * >= 1536 and N < 12800 (K = 14336, N = 4096, 64 rows: 27.9 us against 59.0 us; K = 4096, N = 6144: 18.1 against 34.2);
 * for every other shape and row count the call is w4a16_gemm_stream_bf16 itself and `scratch` is not touched.
 * w4a16_gemm_stream_scratch_bytes(M, K, N) is the scratch the call needs (0 where it takes none): no initialisation,
 * nothing kept between calls, 16-byte aligned; calls that overlap on one GPU need a buffer each.  Same numerics as
 * w4a16_gemm_stream_bf16 below 129 rows (exact weights, fp32 sums, one rounding); the two differ by the order of the
 * fp32 additions only. */
size_t w4a16_gemm_stream_scratch_bytes(int M, int K, int N);
int w4a16_gemm_stream_scratch_bf16(const uint16_t *x, const void *wstream, uint16_t *y, int M, int K, int N, int group,
                                   void *scratch, size_t scratch_bytes, void *stream);
int w4a16_gemv_swiglu_stream_bf16(const uint16_t *x, const void *gate_wstream, const void *up_wstream,
                                  uint16_t *h, int K, int H, int group, void *stream);

/*
 * The rest of the decode path on stream-order matrices; references and rounding points are those of the
 * checkpoint-layout entry points of the same name without `_stream` (declared below), none of these keeps state
 * between calls, and every stage is one whole-K launch.
 * w4a16_rms_gemv_stream_bf16: y = bf16(bf16((x * rstd) * norm_weight) . W), rstd = 1 / sqrt(mean(x^2) + eps); x_sumsq
 *   NULL, or n_pieces (<= 4096) partial sums of x^2 left by the call that produced x (then x is not walked for the
 *   mean; the result agrees up to the summation order of the mean).
 * w4a16_rms_gemv_swiglu_stream_bf16: RMSNorm + gate / up + SwiGLU (matvec_int4_swiglu_rms.cpu_reference,
 *   programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:490-516).
 * w4a16_ffn_swiglu_stream_bf16: h = bf16(silu(bf16(x . Wg)) * bf16(x . Wu)), y = bf16(h . Wd); `h` (bf16 [H]) is
 *   required: it is the intermediate's only home.  Two launches.
 * w4a16_o_gemv_ffn_stream_bf16: the three stages of o_gemv_ffn_int4
 *   (programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_gemv_ffn_int4_multi.py:4-37) as three launches;
 *   res1_out / h_out may be NULL; y_sumsq NULL or E / 16 floats that receive the sum of squares of the bf16 values of y
 *   per 16 columns, which w4a16_rms_gemv_stream_bf16 of the next layer takes as x_sumsq.  The workspace is plain
 *   scratch (no initialisation, nothing kept between calls), w4a16_block_stream_workspace_bytes(E, H).
 * w4a16_decode_attn_o_gemv_ffn_stream_bf16: w4a16_decode_attention_bf16 followed by the block, as one call
 *   (everything of a decode layer after the Q|K|V projection, llama32_1b_int4_decode.py:270-313).
 */
int w4a16_rms_gemv_stream_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                               const void *wstream, uint16_t *y, int K, int N, int group, void *stream);
int w4a16_rms_gemv_swiglu_stream_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, const void *gate_wstream,
                                      const void *up_wstream, uint16_t *h, int K, int H, int group, void *stream);
int w4a16_ffn_swiglu_stream_bf16(const uint16_t *x, const void *gate_wstream, const void *up_wstream,
                                 const void *down_wstream, uint16_t *y, uint16_t *h, int K, int H, int group, void *stream);
size_t w4a16_block_stream_workspace_bytes(int E, int H);
int w4a16_o_gemv_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                 float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                 const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, float *y_sumsq,
                                 int E, int H, int group, void *workspace, size_t workspace_bytes, void *stream);
int w4a16_decode_attn_o_gemv_ffn_stream_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row, uint16_t *k_cache,
                                             uint16_t *v_cache, uint16_t *attn_out, int pos, int max_seq, int n_heads,
                                             int n_kv_heads, int head_dim, void *attn_workspace, size_t attn_workspace_bytes,
                                             const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                             const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                             const void *down_wstream, uint16_t *y, float *y_sumsq, int E, int H, int group,
                                             void *workspace, size_t workspace_bytes, void *stream);

/*
 * RMSNorm prologue + decode GEMV, batch 1:
 *   rstd = 1 / sqrt(mean(x^2) + eps),  n = bf16((x * rstd) * norm_weight),  y = bf16(n . W)
 * The normalisation of matvec_int4_swiglu_rms.cpu_reference
 * (programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:496-500) in front of a
 * plain GEMV (the shape of the Q/K/V projections of rms_qkv_int4_rope_multi.py:4-30).
 * `norm_weight` is bf16 [K].  Workspace: w4a16_gemm_workspace_bytes(1, K, N).
 */
int w4a16_rms_gemv_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps,
                        const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales,
                        uint16_t *y, int K, int N, int group,
                        void *workspace, size_t workspace_bytes, void *stream);

/*
 * RMSNorm + gate/up GEMV + SwiGLU, batch 1: the whole of matvec_int4_swiglu_rms.cpu_reference
 * (programming_examples/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:490-516) =
 * lgu_cpu_reference (programming_examples/llms/llama32_1b_int4/multi_launch_builder/
 * o_gemv_ffn_int4_fused.py:127-151) in one kernel.  Workspace: w4a16_ffn_workspace_bytes(K, H).
 */
int w4a16_rms_gemv_swiglu_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps,
                               const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                               const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                               uint16_t *h, int K, int H, int group,
                               void *workspace, size_t workspace_bytes, void *stream);

/*
 * Decode block "O projection + FFN", batch 1 — the three stages of o_gemv_ffn_int4
 * (programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_gemv_ffn_int4_multi.py:4-37):
 *   res1 = bf16(attn_out . Wo + x_residual)
 *   h    = bf16(silu(bf16(n . Wg)) * bf16(n . Wu)),  n = bf16((res1 * rstd) * ffn_norm_weight)
 *   y    = bf16(h . Wd + res1)
 * Wo is [E, E], Wg and Wu are [E, H], Wd is [H, E]; attn_out, x_residual, ffn_norm_weight, y
 * are bf16 [E].  `res1_out` (bf16 [E]) and `h_out` (bf16 [H]) may be NULL; when given they
 * receive the intermediates.  Three kernel launches on `stream`.
 * Workspace: w4a16_block_workspace_bytes(E, H).
 */
size_t w4a16_block_workspace_bytes(int E, int H);
int w4a16_o_gemv_ffn_bf16(const uint16_t *attn_out, const uint16_t *x_residual,
                          const uint16_t *ffn_norm_weight, float eps,
                          const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                          const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                          const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                          const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                          uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int E, int H, int group,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * Decode attention for one new token with the RoPE of Q and K and the KV-cache append fused in.
 * `qkv` is the token's fresh projection [Q (n_heads * head_dim) | K (n_kv_heads * head_dim) |
 * V (n_kv_heads * head_dim)] bf16, e.g. the output of w4a16_rms_gemv_bf16 on the concatenated
 * Q|K|V weights; `rope_lut_row` is row `pos` of the RoPE table, bf16 [head_dim] = cos then sin
 * (generate_rope_lut, programming_examples/llms/llama32_1b/llama32_1b_weights.py:395-444).
 * The kernel rotates Q and K half-split (rope_halfsplit, _cpu_rope in
 * programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:508-524), writes the
 * rotated K and V into k_cache / v_cache [n_kv_heads, max_seq, head_dim] at `pos`, and computes
 * single-query grouped-query attention over positions 0..pos (decode_attention_cpu,
 * programming_examples/llms/llama32_1b_int4/llama32_1b_int4_decode.py:135-168, which the
 * reference runs on the host CPU) into attn_out bf16 [n_heads * head_dim].
 * Replaces launches L5, L6 of rms_qkv_int4_rope (rms_qkv_int4_rope_multi.py:4-30), the cache
 * update and the attention of run_decode_block (llama32_1b_int4_decode.py:270-285).
 * head_dim 64 or 128; n_heads / n_kv_heads in {1, 2, 4, 8}; 0 <= pos < max_seq.
 * The workspace is plain scratch (no initialisation), w4a16_attention_workspace_bytes().
 */
size_t w4a16_attention_workspace_bytes(int n_heads, int head_dim);

/*
 * w4a16_decode_attention_bf16 followed by w4a16_o_gemv_ffn_bf16 as one call: everything of a decode layer after
 * the Q|K|V projection (RoPE, cache append and attention of run_decode_block, then the o_gemv_ffn_int4 ELF,
 * programming_examples/llms/llama32_1b_int4/llama32_1b_int4_decode.py:270-313).  When the attention runs over
 * several sequence chunks and the O projection's work units lie inside one head (head_dim % 64 == 0 and a short
 * enough E), the O projection merges the chunk partials itself, with the merge kernel's arithmetic in the merge
 * kernel's order, and the merge launch is dropped: y is the same bit for bit as from the two calls.  `attn_out`
 * bf16 [E] is scratch (it holds the attention output whenever the merge launch did run).  E == n_heads * head_dim;
 * other constraints and both workspaces as for the two calls.  w4a16_tune("attn_fuse", 0) keeps the merge launch.
 * y_sumsq (NULL, or E / 256 floats with E % 256 == 0, E <= 16384): receives the sum of squares of the bf16 values
 * of y per 256-column tile, which w4a16_rms_gemv_sumsq_bf16 of the next layer takes in place of its own pass over
 * x: there x_sumsq holds n_pieces (<= 64) partial sums of x^2, and the result is that of w4a16_rms_gemv_bf16 up to
 * the summation order of the mean (the RMSNorm front of rms_qkv_int4_rope, rms_qkv_int4_rope_multi.py:4-30).
 */
int w4a16_rms_gemv_sumsq_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                              const int32_t *qweight, const int32_t *qzeros, const uint16_t *scales, uint16_t *y, int K,
                              int N, int group, void *workspace, size_t workspace_bytes, void *stream);
int w4a16_decode_attn_o_gemv_ffn_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row, uint16_t *k_cache,
                                      uint16_t *v_cache, uint16_t *attn_out, int pos, int max_seq, int n_heads,
                                      int n_kv_heads, int head_dim, void *attn_workspace, size_t attn_workspace_bytes,
                                      const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                      const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                                      const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                                      const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                                      const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                                      uint16_t *y, float *y_sumsq, int E, int H, int group, void *workspace,
                                      size_t workspace_bytes, void *stream);

/*
 * Half-split RoPE on its own, for callers that keep the reference's launch structure (launches L5 and L6
 * of rms_qkv_int4_rope, programming_examples/llms/llama32_1b_int4/multi_launch_builder/rms_qkv_int4_rope_multi.py:4-30):
 *   out[r, i]        = bf16(x[r, i] * cos[r, i] - x[r, i + dim/2] * sin[r, i])
 *   out[r, i + dim/2] = bf16(x[r, i + dim/2] * cos[r, i] + x[r, i] * sin[r, i])          i < dim/2, fp32
 * with lut[r, :] = [cos_0 .. cos_{dim/2-1}, sin_0 .. sin_{dim/2-1}] (one LUT row per row of x, the tiled
 * lut_q / lut_k buffers of that ABI).  Replaces the device kernel
 * rope(bfloat16 *input, bfloat16 *lut, bfloat16 *output, int32_t dims)
 * (programming_examples/rope_halfsplit/rope_halfsplit.cc:86-89); CPU form _cpu_rope
 * (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:508-524).  x, lut, out bf16 [rows, dim],
 * dim % 16 == 0, out may not alias x.
 */
int rope_halfsplit_bf16(const uint16_t *x, const uint16_t *lut, uint16_t *out, int rows, int dim, void *stream);
int w4a16_decode_attention_bf16(const uint16_t *qkv, const uint16_t *rope_lut_row,
                                uint16_t *k_cache, uint16_t *v_cache, uint16_t *attn_out,
                                int pos, int max_seq, int n_heads, int n_kv_heads, int head_dim,
                                void *workspace, size_t workspace_bytes, void *stream);

/*
 * Prefill counterpart of w4a16_o_gemv_ffn_bf16 for M tokens at once: the reference's 8-launch ELF `o_ffn_int4`
 * (programming_examples/llms/llama32_1b_int4/multi_launch_builder/o_ffn_int4_multi.py:4-17; CPU
 * reference :644-665) as four GEMM launches with fused epilogues and one RMSNorm launch:
 *   res1    = bf16(bf16(attn_out . Wo) + x_residual)
 *   normed2 = bf16((res1 / sqrt(mean(res1^2) + eps)) * ffn_norm_weight)      per row, fp32
 *   h       = bf16(silu(bf16(normed2 . Wgate)) * bf16(normed2 . Wup))        silu(g) = g / (1 + exp(-g)), fp32
 *   y       = bf16(bf16(h . Wdown) + res1)
 * attn_out, x_residual, y bf16 [M, E]; optional outputs res1_out [M, E] and h_out [M, H] (NULL: kept
 * in the workspace).  Any M >= 1 (the tiled kernel is used whatever M is), E % 128 == 0,
 * E <= 8192, H % 128 == 0.  The workspace is plain scratch (no initialisation),
 * w4a16_prefill_block_workspace_bytes(M, E, H): 4 M E + 4 M H bytes for res1, normed2, gate and h, plus
 * the fp32 split-K slices (up to 16 M max(E, H) bytes) of the projections that have too few 256 x 256 tiles to
 * fill the GPU.
 * rms_norm_rows_bf16 is the block's RMSNorm stage on its own (the `weighted_rms_norm` launch of both
 * prefill ELFs): out[m, :] = bf16((x[m, :] / sqrt(mean(x[m, :]^2) + eps)) * norm_weight), K % 8 == 0, K <= 8192.
 */
size_t w4a16_prefill_block_workspace_bytes(int M, int E, int H);
int rms_norm_rows_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, uint16_t *out, int M, int K,
                       void *stream);
int w4a16_prefill_o_ffn_bf16(const uint16_t *attn_out, const uint16_t *x_residual,
                             const uint16_t *ffn_norm_weight, float eps,
                             const int32_t *o_qweight, const int32_t *o_qzeros, const uint16_t *o_scales,
                             const int32_t *gate_qweight, const int32_t *gate_qzeros, const uint16_t *gate_scales,
                             const int32_t *up_qweight, const int32_t *up_qzeros, const uint16_t *up_scales,
                             const int32_t *down_qweight, const int32_t *down_qzeros, const uint16_t *down_scales,
                             uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E, int H, int group,
                             void *workspace, size_t workspace_bytes, void *stream);

/*
 * The two prompt-pass blocks on stream-order weights (w4a16_repack_stream of the same matrices; the Q|K|V matrices
 * concatenated along N before the re-pack): w4a16_prefill_rms_qkv_rope_bf16 and w4a16_prefill_o_ffn_bf16 with the tiled
 * stream-order GEMM (w4a16_gemm_stream_bf16's kernel for M >= 129) and its fused epilogues in place of the
 * checkpoint-layout GEMM.  Same references (rms_gemms_rope_int4_multi.py:4-17, 414-436, 543-561;
 * o_ffn_int4_multi.py:4-17, 644-665), same rounding points, same workspaces (w4a16_prefill_qkv_workspace_bytes,
 * w4a16_prefill_block_workspace_bytes; plain scratch).  E % 256 == 0, H % 256 == 0, every N % 64 == 0.
 */
int w4a16_prefill_rms_qkv_rope_stream_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps, const void *qkv_wstream,
                                           const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M, int E,
                                           int n_heads, int n_kv_heads, int head_dim, int group, void *workspace,
                                           size_t workspace_bytes, void *stream);
int w4a16_prefill_o_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight, float eps,
                                    const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                    const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                    int H, int group, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Prefill counterpart of w4a16_rms_gemv_bf16 + the RoPE of w4a16_decode_attention_bf16 for M tokens at
 * positions pos0 .. pos0 + M - 1: the reference's 6-launch ELF `rms_gemms_rope_int4`
 * (programming_examples/llms/llama32_1b_int4/multi_launch_builder/rms_gemms_rope_int4_multi.py:4-17; CPU reference
 * :414-436 and :543-561) as one RMSNorm launch and one GEMM over the Q|K|V weights concatenated along N:
 *   normed   = bf16((x / sqrt(mean(x^2) + eps)) * attn_norm_weight)          per row, fp32
 *   q, k, v  = bf16(normed . Wq), bf16(normed . Wk), bf16(normed . Wv)
 *   q, k     = half-split RoPE per head with row pos0 + m of the table      (_rope_ref; fp32, one rounding)
 * x bf16 [M, E]; qkv_out bf16 [M, (n_heads + 2 n_kv_heads) * head_dim] = Q | K | V per row; rope_lut bf16
 * [rope_lut_rows, head_dim], cos then sin (generate_rope_lut), pos0 + M <= rope_lut_rows.  head_dim 64 or 128,
 * E % 128 == 0, E <= 8192.  The workspace is plain scratch, w4a16_prefill_qkv_workspace_bytes(M, E) = 2 M E bytes.
 */
size_t w4a16_prefill_qkv_workspace_bytes(int M, int E);
int w4a16_prefill_rms_qkv_rope_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps,
                                    const int32_t *qkv_qweight, const int32_t *qkv_qzeros, const uint16_t *qkv_scales,
                                    const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out,
                                    int M, int E, int n_heads, int n_kv_heads, int head_dim, int group,
                                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * Causal grouped-query attention over the M tokens of a prefill: the `flash_attn` step between the two prefill ELFs
 * (programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:302-326; CPU form attention_reference,
 * programming_examples/llms/llama32_1b/llama32_1b_cpu_helpers.py:50-88: softmax(Q K^T / sqrt(head_dim) + causal
 * mask) V per head, query head h reading KV head h / (n_heads / n_kv_heads)).
 * qkv bf16 [M, (n_heads + 2 n_kv_heads) * head_dim] is the output of w4a16_prefill_rms_qkv_rope_bf16 (roped Q | roped
 * K | V per row); attn_out bf16 [M, n_heads * head_dim].  Token m attends to tokens 0..m of the same call (no earlier
 * cache).  fp32 softmax with the probabilities rounded to bf16 for the P.V product.  head_dim 64 or 128.
 */
int w4a16_prefill_attention_bf16(const uint16_t *qkv, uint16_t *attn_out, int M, int n_heads, int n_kv_heads,
                                 int head_dim, void *stream);

/*
 * Tail of a decode step: final RMSNorm, bf16 lm_head GEMV and argmax in one call
 * (run_npu_decode_step, programming_examples/llms/llama32_1b_int4/llama32_1b_int4_inference.py:459-486:
 * host rms_norm, the `lm_head_gemv` kernel over 8 vocabulary partitions, np.argmax).
 *   normed = bf16((x / sqrt(mean(x^2) + eps)) * norm_weight)     fp32 arithmetic (rms_norm,
 *            programming_examples/llms/llama32_1b/llama32_1b_cpu_helpers.py:25-39); norm_weight NULL: normed = x
 *   logits[v] = bf16(sum_e lm_head[v, e] * normed[e])             lm_head bf16 [V, E] row-major, fp32 accumulation
 *   *argmax_out = lowest v with the largest logit                 (may be NULL; a NaN logit counts as the largest if positive)
 * x bf16 [E], logits bf16 [V] (every V >= 1; the reference pads the vocabulary to 8 x 16384 rows
 * instead).  E % 8 == 0, E <= 8192.  The workspace is plain scratch
 * (no initialisation), lm_head_workspace_bytes(V).
 */
size_t lm_head_workspace_bytes(int V);
int lm_head_gemv_bf16(const uint16_t *x, const uint16_t *norm_weight, float eps, const uint16_t *lm_head,
                      uint16_t *logits, int32_t *argmax_out, int V, int E,
                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * Q4NX / Q4_0 block codec (the 4-bit formats of the fused decode examples).  W[M, K] (M output
 * features, K input features) is stored as (M / 32) x (K / 256) blocks of 5120 bytes, row-block
 * major, each holding bf16 scales[8][32], bf16 mins[8][32] (one per row and 32-column group) and
 * the nibbles qs[2][256][8] with byte kk of (rg, col) = (q[16 rg + 2 kk + 1][col] << 4) |
 * q[16 rg + 2 kk][col] (pack_q4k_block, programming_examples/fused_decode/proj_qmm_pack.py:4-58;
 * q4k_block_t, programming_examples/fused_decode/kernels/model_spec.h:86-103).
 * `mode` selects the value convention:
 *   W4A16_Q4NX_ADDITIVE     w = s * q + m, q unsigned: what the proj_qmm kernel computes
 *                           (programming_examples/fused_decode/kernels/q4_k.h:9-17) and what bundles
 *                           with an "I8" header hold (Q4nxModel.dequant,
 *                           programming_examples/llms/llama32_1b_q4nx/llama32_1b_q4nx_weights.py:205-266)
 *   W4A16_Q4NX_SUBTRACTIVE  w = s * (q - m): bundles with a "Q4NX" header (same function, :255-261)
 *   W4A16_Q4_0              w = s * q, q signed two's complement, mins ignored
 *                           (programming_examples/fused_decode/qwen25_3b_requant.py:13-17, 116-134)
 *
 * q4nx_dequant_bf16 writes the dense matrix out[M, K] = bf16(w) (fp32 arithmetic in the order
 * written above, one rounding to bf16), replacing Q4nxModel.dequant / dequant_q4_0
 * (programming_examples/llms/qwen25_3b_q4/qwen25_3b_q4_weights.py:86-95) followed by the cast to bf16.
 *
 * q4nx_repack turns the blocks into the operands of w4a16_q4nx_repack_stream, once at load time (the
 * reference re-packs the same blocks into its own device stream order, pack_q4k_cascade,
 * proj_qmm_pack.py:61-140): qweight int32 [K, M / 8] (word (k, j) = rows 8 j .. 8 j + 7 of
 * column k, unsigned nibbles in the AutoAWQ order), scales and mins bf16 [K / 32, M] with
 * w = q * scale + min.  W4A16_Q4_0 is exact (q ^ 8, min = -8 s); W4A16_Q4NX_SUBTRACTIVE stores
 * min = bf16(-s * m), one extra rounding of the constant term.
 * M % 32 == 0, K % 256 == 0, all pointers 16-byte aligned.
 */
#define W4A16_Q4NX_ADDITIVE 0
#define W4A16_Q4NX_SUBTRACTIVE 1
#define W4A16_Q4_0 2
int q4nx_dequant_bf16(const void *blocks, uint16_t *out_bf16, int M, int K, int mode, void *stream);
int q4nx_repack(const void *blocks, int32_t *qweight, uint16_t *scales, uint16_t *mins,
                int M, int K, int mode, void *stream);

/*
 * The products of this codec: the operands of q4nx_repack re-packed once more, at load time, into the stream order of
 * the decode kernels (csrc/wstream.h, "Q4NX order": 16-column tiles, 1 KiB cells of 128 rows, and in front of every 16
 * cells 4 KiB of scale / min words, one pair per 32 rows and column), the counterpart of the reference's own stream
 * order for these blocks (pack_q4k_cascade, programming_examples/fused_decode/proj_qmm_pack.py:61-140).  The GEMV, the
 * RMSNorm + GEMV and the O + FFN block then run the whole-K kernels of the AWQ stream order with the per-32-row flush
 * y += s * (sum q x) + min * (sum x) of _qmm_q4k_bf16 (programming_examples/fused_decode/kernels/q4_k.h:39-45: c += (q*b)*scale;
 * c += min*sum(b)): no workspace protocol, no state.  They cover the proj / O / FFN phases of the fused decode dispatch
 * (programming_examples/fused_decode/fused_decode.py: proj_qmm, rms_residual, glu kernels) around w4a16_decode_attention_bf16; the
 * reference runs the prefill of these models as dense bf16 GEMMs on dequantised weights; the large-M entry points below multiply the same bf16 values without leaving the codec.  `residual` may be NULL; x_sumsq / n_pieces, res1_out, h_out, y_sumsq and the workspace
 * (w4a16_block_stream_workspace_bytes) as in the AWQ entry points of the same names.  K % 128 == 0, N % 16 == 0.
 */
size_t w4a16_q4nx_stream_bytes(int K, int N);
/* Blocks of W[M, K] (uint8 [M / 32 * K / 256, 5120], as q4nx_dequant_bf16 takes them) -> the Q4NX order of the [K, N = M]
 * matrix in one pass: the same bytes as q4nx_repack followed by w4a16_q4nx_repack_stream, without the intermediate
 * operands; the one load-time re-pack of the reference's packer (programming_examples/fused_decode/proj_qmm_pack.py:61-140).
 * `wstream`: w4a16_q4nx_stream_bytes(K, M) bytes.  M % 32 == 0, K % 256 == 0, mode as for q4nx_repack. */
int w4a16_q4nx_blocks_to_stream(const void *blocks, void *wstream, int M, int K, int mode, void *stream);
int w4a16_q4nx_repack_stream(const int32_t *qweight, const uint16_t *scales, const uint16_t *mins, void *wstream, int K, int N,
                             void *stream);
int w4a16_q4nx_gemv_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual, uint16_t *y, int K, int N,
                                void *stream);
/* y[M, N] = bf16(x[M, K] . W + residual [M, N]): the GEMV at M = 1, the batched whole-K kernel in launches of 16 rows
 * above (exact weights s q + min', fp32 sums, one rounding).  From M = 65 on, without a residual and with K % 256 == 0,
 * N % 64 == 0, the tiled MFMA kernel of w4a16_gemm_stream_bf16 runs on the Q4NX order: it dequantises each K-step of a
 * cell with its own (scale, min') word to W = bf16_rne(s q + min'), the dense dequant's values (q4nx_dequant_bf16,
 * bit for bit), and multiplies those, which is what the reference's prompt pass of these models computes with its
 * dense bf16 GEMMs on dequantised weights (programming_examples/llms/llama31_8b_q4nx/README.md:11-15). */
int w4a16_q4nx_gemm_stream_bf16(const uint16_t *x, const void *wstream, const uint16_t *residual, uint16_t *y, int M, int K, int N,
                                void *stream);
/* The two prompt-pass blocks (w4a16_prefill_rms_qkv_rope_stream_bf16, w4a16_prefill_o_ffn_stream_bf16: same arguments
 * without `group`, same stages, rounding points and workspaces) on matrices in Q4NX order: the reference runs these
 * stages op by op as bf16 GEMM / RMSNorm / RoPE / SwiGLU on the dequantised weights
 * (programming_examples/llms/llama31_8b_q4nx/README.md:11-15); here the weights stay at 5 bits and are dequantised in
 * registers to the same bf16 values. */
int w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16(const uint16_t *x, const uint16_t *attn_norm_weight, float eps, const void *qkv_wstream,
                                                const uint16_t *rope_lut, int rope_lut_rows, int pos0, uint16_t *qkv_out, int M,
                                                int E, int n_heads, int n_kv_heads, int head_dim, void *workspace,
                                                size_t workspace_bytes, void *stream);
int w4a16_q4nx_prefill_o_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                         float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                         const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, int M, int E,
                                         int H, void *workspace, size_t workspace_bytes, void *stream);
int w4a16_q4nx_rms_gemv_stream_bf16(const uint16_t *x, const float *x_sumsq, int n_pieces, const uint16_t *norm_weight, float eps,
                                    const void *wstream, uint16_t *y, int K, int N, void *stream);
int w4a16_q4nx_o_gemv_ffn_stream_bf16(const uint16_t *attn_out, const uint16_t *x_residual, const uint16_t *ffn_norm_weight,
                                      float eps, const void *o_wstream, const void *gate_wstream, const void *up_wstream,
                                      const void *down_wstream, uint16_t *y, uint16_t *res1_out, uint16_t *h_out, float *y_sumsq,
                                      int E, int H, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Launch-shape override for benchmarking sweeps (not needed for normal use).  Keys:
 * "gemv_lw", "gemv_ksteps", "gemv_waves", "gemv_units", "gemv_ksplit" (0 = built-in heuristic),
 * "gemm_stream_max_m" (largest M given to the streaming kernel, 0 = default 96, otherwise >= 16) and
 * "gemv_spin_limit" (reducer poll bound), "gemv_skip_publish" (fault injection for the
 * timeout test: split-K producers do not publish), "gemv_ws_ct", "gemv_ws_waves",
 * "gemm_ws_cb", "gemm_ws_rows" (stream-order GEMV / small-batch shapes; rows: most rows per batched launch, 16, 32 or 64), "prefill_tile" (one tile width only, 1: 256 columns, 2: 192, 3: 128,
 * 4: 64; 5: 256 mixed with 128 in the launches that take that mix; 0: by shape), "prefill_min_m" (smallest M given to the tiled prefill kernel), "prefill_band" (row panels per band of its tile order), "gemm_splitk" (w4a16_gemm_stream_scratch_bf16 at 17 .. 128 rows: 0 split along K by shape, 1 always, 2 never) and "prefill_swiglu_split" (1: the
 * stream-order prompt-pass FFN runs its gate and up projections as two launches instead of one; same bits).  Process-wide.
 */
int w4a16_tune(const char *key, int value);

#ifdef __cplusplus
}
#endif
#endif /* W4A16_H */
