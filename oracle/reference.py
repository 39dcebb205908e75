"""TEST INFRASTRUCTURE ONLY - CPU restatement of the examples' cpu_reference
functions for the W4A16 path.  Never imported by the product.

Follows (PE = programming_examples, INT4 = PE/llms/llama32_1b_int4):

  matvec_cpu_reference_loop  PE/matrix_vector_multiplication/int4_awq/
                             matvec_int4_packed.py:272-287 (scalar double loop;
                             each term is a double under NumPy promotion and the
                             running sum is re-rounded to float32 every step)
  matvec_cpu_reference       same sum with float64 accumulation (vectorised as
                             PE/decode_ffn_swiglu/matvec_int4_swiglu_rms.py:501-511)
  matvec_add_cpu_reference   .../int4_awq/matvec_int4_packed_add.py:302-319
  matmul_cpu_reference       PE/matrix_multiplication/int4_awq/
                             matmul_int4_packed.py:89-105
  swiglu_rms_cpu_reference   matvec_int4_swiglu_rms.py:490-516
                             (= lgu_cpu_reference,
                             INT4/multi_launch_builder/o_gemv_ffn_int4_fused.py:127-151)
  ld_cpu_reference           o_gemv_ffn_int4_fused.py:1078-1094
  ffn_swiglu_reference       the chain at o_gemv_ffn_int4_fused.py:1187-1191
                             without the RMSNorm prologue and with R = 0
  o_gemv_ffn_int4_reference  INT4/multi_launch_builder/o_gemv_ffn_int4_multi.py:273-288
                             (float32 throughout on bf16-dequantised weights; res1
                             and gate/up are NOT rounded to bf16)
  o_gemv_ffn_staged_reference  the three device stages of the same block
                             (o_gemv_ffn_int4_multi.py:4-37) chained with the
                             per-stage references above, i.e. with the bf16
                             rounding points the stages have on the device
  o_ffn_int4_prefill_reference  the CPU reference of the 8-launch prefill ELF
                             (INT4/multi_launch_builder/o_ffn_int4_multi.py:644-665): four
                             matmul_cpu_reference products with bf16 outputs, residual adds
                             and the row-wise RMSNorm in float32 (r1 / rms * w), SwiGLU
                             with silu(g) = g / (1 + exp(-g)) in float32
  check_outputs              python/air/backend/xrt_runner.py:394-523

Arrays named A_q/A_s/A_z use the examples' kernel-side layout
(A_q u8 [out, K/2], A_s bf16 bits [K/gs, out], A_z u8 [K/gs, out]); bf16
tensors are uint16 bit patterns.

The scalar loop also exists in C (oracle/w4a16_oracle.c) so that it can be run
at full size; tests/test_oracle_reference.py checks the C build against this
Python loop on small shapes and both against closed forms (one-hot x, z=0 s=1
integer matrices, constant-q groups).
"""

import numpy as np

from .awq import l1_unpack_nibbles
from .bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def _dequant_l1_f64(a_q, a_s_bits, a_z, k):
    """(nib - z) * s as the vectorised references build it: int32 * float32
    arrays promote to float64; shape [out, K]."""
    n_groups = a_s_bits.shape[0]
    gs = k // n_groups
    nibs = l1_unpack_nibbles(a_q)
    s_per_kk = np.repeat(bf16_bits_to_f32(a_s_bits), gs, axis=0)
    z_per_kk = np.repeat(np.asarray(a_z).astype(np.int32), gs, axis=0)
    return (nibs - z_per_kk.T).astype(np.float64) * s_per_kk.T.astype(np.float64)


def matvec_cpu_reference_loop(a_q, a_s_bits, a_z, b_bits):
    """Scalar restatement; use only on small shapes (pure Python)."""
    m = a_q.shape[0]
    k = b_bits.shape[0]
    n_groups = a_s_bits.shape[0]
    gs = k // n_groups
    d = np.zeros(m, dtype=np.float32)
    bf = bf16_bits_to_f32(b_bits)
    s_f = bf16_bits_to_f32(a_s_bits)
    z_i = np.asarray(a_z).astype(np.int32)
    for r in range(m):
        for kk in range(k):
            byte = int(a_q[r, kk // 2])
            nib = (byte & 0x0F) if (kk % 2 == 0) else ((byte >> 4) & 0x0F)
            g = kk // gs
            term = float(nib - int(z_i[g, r])) * float(s_f[g, r]) * float(bf[kk])
            d[r] = np.float32(float(d[r]) + term)
    return f32_to_bf16_bits(d)


def matvec_f64(a_q, a_s_bits, a_z, b_bits):
    """Exact-term, float64-accumulated GEMV; returns float64 [out]."""
    k = b_bits.shape[0]
    dq = _dequant_l1_f64(a_q, a_s_bits, a_z, k)
    return dq @ bf16_bits_to_f32(b_bits).astype(np.float64)


def matvec_cpu_reference(a_q, a_s_bits, a_z, b_bits):
    return f32_to_bf16_bits(matvec_f64(a_q, a_s_bits, a_z, b_bits).astype(np.float32))


def matvec_add_cpu_reference(a_q, a_s_bits, a_z, b_bits, r_bits):
    """D = bf16(float32(sum) + R): the residual joins the float32 sum before
    the single bf16 rounding."""
    acc = matvec_f64(a_q, a_s_bits, a_z, b_bits).astype(np.float32)
    return f32_to_bf16_bits(acc + bf16_bits_to_f32(r_bits))


def matmul_cpu_reference(w_q, w_s_bits, w_z, a_bits, round_weights=False, accumulate="f32"):
    """C[M, N] = bf16(A @ W_dq); W_dq[k, n] = (nib - z) * s kept in float32.

    round_weights=True rounds W_dq to bf16 first (the weights a kernel that
    dequantises to bf16 tiles actually multiplies).  accumulate="f64" uses a
    float64 product, "f32" the reference's float32 BLAS product.
    """
    k = a_bits.shape[1]
    w_dq = _dequant_l1_f64(w_q, w_s_bits, w_z, k).T.astype(np.float32)  # [K, N], exact
    if round_weights:
        w_dq = bf16_bits_to_f32(f32_to_bf16_bits(w_dq))
    af = bf16_bits_to_f32(a_bits)
    if accumulate == "f64":
        c = (af.astype(np.float64) @ w_dq.astype(np.float64)).astype(np.float32)
    else:
        c = af @ w_dq
    return f32_to_bf16_bits(c)


def silu_tanh_f32(gate):
    """silu(g) = g * 0.5 * (tanh(g / 2) + 1) in float32."""
    gate = np.asarray(gate, dtype=np.float32)
    return gate * np.float32(0.5) * (np.tanh(gate / np.float32(2.0)) + np.float32(1.0))


def rms_norm_bf16(x_bits, w_bits, eps=1e-5):
    """normed = bf16((x * rstd) * w) as float32 values."""
    x = bf16_bits_to_f32(x_bits)
    w = bf16_bits_to_f32(w_bits)
    mean_sq = float((x * x).sum()) / x.shape[0]
    rstd = 1.0 / np.sqrt(mean_sq + eps)
    normed = ((x * rstd) * w).astype(np.float32)
    return bf16_bits_to_f32(f32_to_bf16_bits(normed))


def swiglu_rms_cpu_reference(a_q, a_s_bits, a_z, x_bits, norm_w_bits=None, eps=1e-5):
    """Interleaved gate/up GEMV + SwiGLU; rows 2i = gate, 2i+1 = up; output
    bf16 bits [out/2].  norm_w_bits=None skips the RMSNorm prologue."""
    k = x_bits.shape[0]
    if norm_w_bits is None:
        normed = bf16_bits_to_f32(x_bits)
    else:
        normed = rms_norm_bf16(x_bits, norm_w_bits, eps)
    raw = _dequant_l1_f64(a_q, a_s_bits, a_z, k) @ normed.astype(np.float64)
    raw_bf16 = bf16_bits_to_f32(f32_to_bf16_bits(raw.astype(np.float32)))
    gate = raw_bf16[0::2]
    up = raw_bf16[1::2]
    return f32_to_bf16_bits(silu_tanh_f32(gate) * up)


def ld_cpu_reference(a_q, a_s_bits, a_z, swiglu_bits, r_bits=None):
    """D = bf16(bf16(dequant @ swiglu) + R)."""
    k = swiglu_bits.shape[0]
    raw = _dequant_l1_f64(a_q, a_s_bits, a_z, k) @ bf16_bits_to_f32(swiglu_bits).astype(np.float64)
    raw_bits = f32_to_bf16_bits(raw.astype(np.float32))
    if r_bits is None:
        return raw_bits
    return f32_to_bf16_bits(bf16_bits_to_f32(raw_bits) + bf16_bits_to_f32(r_bits))


def interleave_gate_up(gate_l1, up_l1):
    """Row-interleave two kernel-side weight triples: row 2i = gate[i],
    row 2i+1 = up[i] (INT4/llama32_1b_int4_weights.py:173-207)."""
    gq, gs_, gz = gate_l1
    uq, us_, uz = up_l1
    out = gq.shape[0]
    a_q = np.empty((2 * out, gq.shape[1]), dtype=np.uint8)
    a_q[0::2] = gq
    a_q[1::2] = uq
    a_s = np.empty((gs_.shape[0], 2 * out), dtype=np.uint16)
    a_s[:, 0::2] = gs_
    a_s[:, 1::2] = us_
    a_z = np.empty((gz.shape[0], 2 * out), dtype=np.uint8)
    a_z[:, 0::2] = gz
    a_z[:, 1::2] = uz
    return a_q, a_s, a_z


def ffn_swiglu_reference(gate_l1, up_l1, down_l1, x_bits):
    """Decode FFN without norm/residual: returns (h bits [H], y bits [K])."""
    a_q, a_s, a_z = interleave_gate_up(gate_l1, up_l1)
    h = swiglu_rms_cpu_reference(a_q, a_s, a_z, x_bits, None)
    y = ld_cpu_reference(down_l1[0], down_l1[1], down_l1[2], h, None)
    return h, y


def o_gemv_ffn_int4_reference(wo_bits, attn_out_bits, x_residual_bits, ffn_norm_w_bits, wgate_bits, wup_bits,
                              wdown_bits, eps=1e-5):
    """Whole O + FFN block on bf16-dequantised weights ([out, in] bf16 bits), float32
    arithmetic; returns bf16 bits [emb]."""
    f = bf16_bits_to_f32
    res1 = f(wo_bits) @ f(attn_out_bits) + f(x_residual_bits)
    rstd = 1.0 / np.sqrt((res1 * res1).mean() + eps)
    normed = (res1 * rstd) * f(ffn_norm_w_bits)
    normed_bf16 = f(f32_to_bf16_bits(normed.astype(np.float32)))
    gate = f(wgate_bits) @ normed_bf16
    up = f(wup_bits) @ normed_bf16
    swiglu = (gate * 0.5 * (np.tanh(gate / 2.0) + 1.0)) * up
    swiglu_bf16 = f(f32_to_bf16_bits(swiglu.astype(np.float32)))
    return f32_to_bf16_bits((f(wdown_bits) @ swiglu_bf16 + res1).astype(np.float32))


def o_gemv_ffn_staged_reference(wo_l1, gate_l1, up_l1, down_l1, attn_out_bits, x_residual_bits, ffn_norm_w_bits,
                                eps=1e-5):
    """Stage 1 matvec_add, stage 2 RMSNorm + gate/up + SwiGLU, stage 3 matvec_add with
    res1 as the residual.  Returns (res1 bits [emb], h bits [hidden], y bits [emb])."""
    res1 = matvec_add_cpu_reference(wo_l1[0], wo_l1[1], wo_l1[2], attn_out_bits, x_residual_bits)
    a_q, a_s, a_z = interleave_gate_up(gate_l1, up_l1)
    h = swiglu_rms_cpu_reference(a_q, a_s, a_z, res1, ffn_norm_w_bits, eps)
    y = matvec_add_cpu_reference(down_l1[0], down_l1[1], down_l1[2], h, res1)
    return res1, h, y


def rms_norm_rows_bf16(x_bits, w_bits, eps=1e-5):
    """bf16 bits of r / sqrt(mean(r^2, axis=-1) + eps) * w, row-wise, every step in float32."""
    r = bf16_bits_to_f32(np.asarray(x_bits)).astype(np.float32)
    rms = np.sqrt(np.mean(r**2, axis=-1, keepdims=True) + np.float32(eps))
    return f32_to_bf16_bits((r / rms * bf16_bits_to_f32(np.asarray(w_bits)).astype(np.float32)).astype(np.float32))


def o_ffn_int4_prefill_reference(wo_l1, gate_l1, up_l1, down_l1, attn_out_bits, x_residual_bits, ffn_norm_w_bits,
                                 eps=1e-5, **matmul_kw):
    """(output, res1, swiglu) as bf16 bits [M, E], [M, E], [M, H]; every weight is (A_q, A_s, A_z).
    matmul_kw goes to matmul_cpu_reference (round_weights / accumulate)."""
    proj = matmul_cpu_reference(*wo_l1, attn_out_bits, **matmul_kw)
    res1 = f32_to_bf16_bits(bf16_bits_to_f32(proj).astype(np.float32) + bf16_bits_to_f32(x_residual_bits).astype(np.float32))
    normed2 = rms_norm_rows_bf16(res1, ffn_norm_w_bits, eps)
    gate = matmul_cpu_reference(*gate_l1, normed2, **matmul_kw)
    up = matmul_cpu_reference(*up_l1, normed2, **matmul_kw)
    g = bf16_bits_to_f32(gate).astype(np.float32)
    swiglu = f32_to_bf16_bits((g / (np.float32(1.0) + np.exp(-g)) * bf16_bits_to_f32(up).astype(np.float32)).astype(np.float32))
    down = matmul_cpu_reference(*down_l1, swiglu, **matmul_kw)
    out = f32_to_bf16_bits(bf16_bits_to_f32(down).astype(np.float32) + bf16_bits_to_f32(res1).astype(np.float32))
    return out, res1, swiglu


def check_outputs(actual, expected, rtol=1e-3, atol=1e-8, max_mismatch_percentage=0, min_correlation=None):
    """The examples' comparator on float arrays: np.isclose mask, mismatch
    budget int(total * pct / 100), optional Pearson correlation gate."""
    actual = np.reshape(np.asarray(actual, dtype=np.float64), np.shape(expected))
    expected = np.asarray(expected, dtype=np.float64)
    close = np.isclose(actual, expected, rtol=rtol, atol=atol)
    mismatches = int((~close).sum())
    ok = mismatches <= int(expected.size * max_mismatch_percentage / 100)
    if min_correlation is not None and expected.size > 0:
        corr = float(np.corrcoef(actual.flatten(), expected.flatten())[0, 1])
        if not np.isfinite(corr) or corr < min_correlation:
            ok = False
    return ok
