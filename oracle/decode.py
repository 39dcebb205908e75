"""TEST INFRASTRUCTURE ONLY - CPU restatement of the int4 decode block around the W4A16 GEMVs.
Never imported by the product.

Follows (LLM = programming_examples/llms):

  generate_rope_lut      LLM/llama32_1b/llama32_1b_weights.py:395-444 (float64 angles,
                         [cos_0..cos_{h-1}, sin_0..sin_{h-1}] per position, one rounding to bf16)
  rope_halfsplit         LLM/llama32_1b_int4/llama32_1b_int4_prefill.py:508-524 (_cpu_rope):
                         out[i] = x[i] cos[i] - x[i+h] sin[i], out[i+h] = x[i+h] cos[i] + x[i] sin[i]
                         in float32, one rounding to bf16
  decode_attention_cpu   LLM/llama32_1b_int4/llama32_1b_int4_decode.py:135-168 (single-query GQA
                         attention over the KV cache, float32, softmax with max subtraction)
  rms_qkv_rope_reference the six launches of rms_qkv_int4_rope
                         (LLM/llama32_1b_int4/multi_launch_builder/rms_qkv_int4_rope_multi.py:4-30):
                         RMSNorm -> Q, K, V int4 GEMVs -> RoPE on Q and K
  decode_block_reference run_decode_block (llama32_1b_int4_decode.py:176-313): the call above,
                         KV-cache append, attention, then the O + FFN block

  rope_rows, prefill_rms_qkv_rope_reference
                         the CPU reference of the 6-launch prefill ELF rms_gemms_rope_int4
                         (LLM/llama32_1b_int4/multi_launch_builder/rms_gemms_rope_int4_multi.py:414-436,
                         543-561): row-wise RMSNorm to bf16, three matmul_int4_packed products to bf16,
                         half-split RoPE of every Q and K head with the LUT row of the token's position
  prefill_attention_reference  attention_reference (LLM/llama32_1b/llama32_1b_cpu_helpers.py:50-88): causal GQA
                         attention over the tokens of a prefill, float32 softmax per head
  lm_head_reference      the tail of run_npu_decode_step
                         (LLM/llama32_1b_int4/llama32_1b_int4_inference.py:459-486): host rms_norm
                         in float32 (LLM/llama32_1b/llama32_1b_cpu_helpers.py:25-39,
                         (x / sqrt(mean(x^2) + eps)) * w), one rounding to bf16, the bf16
                         lm_head GEMV with bf16 logits, np.argmax over the logits as float32

bf16 tensors are uint16 bit patterns.  Pins (tests/test_oracle_decode.py): RoPE against a complex
rotation and its norm/inverse identities; the LUT against closed forms (pos 0, index 0); attention
against torch's scaled_dot_product_attention and the closed forms seq_len = 1 and equal keys; the
per-row RoPE against the complex rotation by the position's angles and, for equal LUT rows, against
rope_halfsplit; the prefill QKV reference against its stages and the decode-step reference row by row; the
lm_head tail against torch's rms_norm and matmul in float64, one-hot rows (logits = the normalised
vector), a constant vector (closed-form norm) and tied rows (first index wins).
"""

import numpy as np

from .bf16 import bf16_bits_to_f32, f32_to_bf16_bits
from . import reference as ref


def generate_rope_lut(head_dim, rope_base, seq_len):
    """bf16 bits [seq_len, head_dim]: cos of pos * base^(-2i/head_dim) for i < head_dim/2, then sin."""
    half = head_dim // 2
    inv_freq = 1.0 / (rope_base ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim))
    angles = np.outer(np.arange(seq_len, dtype=np.float64), inv_freq)
    lut = np.empty((seq_len, head_dim), dtype=np.float64)
    lut[:, :half] = np.cos(angles)
    lut[:, half:] = np.sin(angles)
    return f32_to_bf16_bits(lut.astype(np.float32))


def rope_halfsplit(x_bits, lut_row_bits):
    """x bf16 bits [rows, dim], one LUT row bf16 bits [dim] shared by all rows -> bf16 bits [rows, dim]."""
    x = bf16_bits_to_f32(x_bits)
    lut = bf16_bits_to_f32(lut_row_bits)
    half = x.shape[1] // 2
    cos, sin = lut[:half], lut[half:]
    x1, x2 = x[:, :half], x[:, half:]
    out = np.empty_like(x)
    out[:, :half] = x1 * cos - x2 * sin
    out[:, half:] = x2 * cos + x1 * sin
    return f32_to_bf16_bits(out)


def decode_attention_cpu(q_bits, k_cache_bits, v_cache_bits, current_pos, n_heads, n_kv_heads, head_dim):
    """q bf16 bits [n_heads * head_dim]; caches bf16 bits [n_kv_heads, max_seq, head_dim] valid up to
    current_pos -> bf16 bits [n_heads * head_dim]."""
    group = n_heads // n_kv_heads
    scale = np.float32(1.0 / np.sqrt(head_dim))
    seq_len = current_pos + 1
    q = bf16_bits_to_f32(q_bits).reshape(n_heads, head_dim)
    k = bf16_bits_to_f32(k_cache_bits[:, :seq_len, :])
    v = bf16_bits_to_f32(v_cache_bits[:, :seq_len, :])
    out = np.zeros((n_heads, head_dim), dtype=np.float32)
    for h in range(n_heads):
        kv = h // group
        scores = (q[h] @ k[kv].T) * scale
        probs = np.exp(scores - scores.max())
        probs = probs / probs.sum()
        out[h] = probs @ v[kv]
    return f32_to_bf16_bits(out.reshape(-1))


def rms_qkv_rope_reference(x_bits, norm_w_bits, wq_l1, wk_l1, wv_l1, lut_row_bits, n_heads, n_kv_heads, head_dim,
                           eps=1e-5):
    """Returns (q_roped bits [n_heads * hd], k_roped bits [n_kv * hd], v bits [n_kv * hd])."""
    normed = f32_to_bf16_bits(ref.rms_norm_bf16(x_bits, norm_w_bits, eps))
    q = ref.matvec_cpu_reference(*wq_l1, normed)
    k = ref.matvec_cpu_reference(*wk_l1, normed)
    v = ref.matvec_cpu_reference(*wv_l1, normed)
    q_r = rope_halfsplit(q.reshape(n_heads, head_dim), lut_row_bits).reshape(-1)
    k_r = rope_halfsplit(k.reshape(n_kv_heads, head_dim), lut_row_bits).reshape(-1)
    return q_r, k_r, v


def decode_block_reference(x_bits, layer_l1, k_cache_bits, v_cache_bits, current_pos, rope_lut_bits, n_heads,
                           n_kv_heads, head_dim, eps=1e-5):
    """One transformer block for one decode token.  `layer_l1` maps attn_norm / ffn_norm to bf16
    bits and wq, wk, wv, wo, w_gate, w_up, w_down to kernel-side triples.  The caches are updated
    in place at current_pos.  Returns the block output bits [emb]."""
    q_r, k_r, v = rms_qkv_rope_reference(x_bits, layer_l1["attn_norm"], layer_l1["wq"], layer_l1["wk"],
                                         layer_l1["wv"], rope_lut_bits[current_pos], n_heads, n_kv_heads, head_dim, eps)
    k_cache_bits[:, current_pos, :] = k_r.reshape(n_kv_heads, head_dim)
    v_cache_bits[:, current_pos, :] = v.reshape(n_kv_heads, head_dim)
    attn = decode_attention_cpu(q_r, k_cache_bits, v_cache_bits, current_pos, n_heads, n_kv_heads, head_dim)
    _, _, y = ref.o_gemv_ffn_staged_reference(layer_l1["wo"], layer_l1["w_gate"], layer_l1["w_up"], layer_l1["w_down"],
                                              attn, x_bits, layer_l1["ffn_norm"], eps)
    return y


def final_rms_norm(x_bits, w_bits, eps=1e-5):
    """bf16 bits of (x / sqrt(mean(x^2) + eps)) * w, every step in float32 as in the host helper."""
    x = bf16_bits_to_f32(np.asarray(x_bits)).astype(np.float32)
    w = bf16_bits_to_f32(np.asarray(w_bits)).astype(np.float32)
    rms = np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + np.float32(eps))
    return f32_to_bf16_bits(((x / rms) * w).astype(np.float32))


def lm_head_reference(x_bits, final_norm_bits, lm_head_bits, eps=1e-5):
    """(logits bf16 bits [V], argmax).  final_norm_bits None: x is used as it is.  The product is
    accumulated in float64 and rounded once (through float32) to bf16."""
    normed = np.asarray(x_bits) if final_norm_bits is None else final_rms_norm(x_bits, final_norm_bits, eps)
    w = bf16_bits_to_f32(np.asarray(lm_head_bits)).astype(np.float64)
    acc = w @ bf16_bits_to_f32(normed).astype(np.float64)
    logits = f32_to_bf16_bits(acc.astype(np.float32))
    return logits, int(np.argmax(bf16_bits_to_f32(logits).astype(np.float32)))


def rope_rows(x_bits, lut_bits):
    """x bf16 bits [rows, dim] rotated with its own LUT row each (lut bf16 bits [rows, dim], cos then sin)."""
    x = bf16_bits_to_f32(np.asarray(x_bits)).astype(np.float32)
    lut = bf16_bits_to_f32(np.asarray(lut_bits)).astype(np.float32)
    half = x.shape[1] // 2
    cos, sin = lut[:, :half], lut[:, half:]
    x1, x2 = x[:, :half], x[:, half:]
    out = np.empty_like(x)
    out[:, :half] = x1 * cos - x2 * sin
    out[:, half:] = x2 * cos + x1 * sin
    return f32_to_bf16_bits(out)


def prefill_rms_qkv_rope_reference(x_bits, norm_w_bits, wq_l1, wk_l1, wv_l1, lut_bits, pos0, n_heads, n_kv_heads,
                                   head_dim, eps=1e-5, **matmul_kw):
    """bf16 bits [M, (n_heads + 2 n_kv_heads) * head_dim] = roped Q | roped K | V for tokens at positions pos0.."""
    M = np.asarray(x_bits).shape[0]
    normed = ref.rms_norm_rows_bf16(x_bits, norm_w_bits, eps)
    q = ref.matmul_cpu_reference(*wq_l1, normed, **matmul_kw)
    k = ref.matmul_cpu_reference(*wk_l1, normed, **matmul_kw)
    v = ref.matmul_cpu_reference(*wv_l1, normed, **matmul_kw)
    rows = np.asarray(lut_bits)[pos0:pos0 + M]
    q = rope_rows(q.reshape(M * n_heads, head_dim), np.repeat(rows, n_heads, axis=0)).reshape(M, -1)
    k = rope_rows(k.reshape(M * n_kv_heads, head_dim), np.repeat(rows, n_kv_heads, axis=0)).reshape(M, -1)
    return np.concatenate([q, k, v], axis=1)


def prefill_attention_reference(q_bits, k_bits, v_bits, n_heads, n_kv_heads):
    """q [M, n_heads * hd], k, v [M, n_kv_heads * hd] bf16 bits -> float32 [M, n_heads * hd]."""
    q, k, v = (bf16_bits_to_f32(np.asarray(t)).astype(np.float32) for t in (q_bits, k_bits, v_bits))
    M = q.shape[0]
    hd = q.shape[1] // n_heads
    group = n_heads // n_kv_heads
    q = q.reshape(M, n_heads, hd).transpose(1, 0, 2)
    k = k.reshape(M, n_kv_heads, hd).transpose(1, 0, 2)
    v = v.reshape(M, n_kv_heads, hd).transpose(1, 0, 2)
    scale = np.float32(1.0 / np.sqrt(hd))
    mask = np.triu(np.full((M, M), -np.inf, dtype=np.float32), k=1)
    out = np.empty((n_heads, M, hd), dtype=np.float32)
    for h in range(n_heads):
        scores = q[h] @ k[h // group].T * scale + mask
        probs = np.exp(scores - scores.max(axis=-1, keepdims=True))
        probs = probs / probs.sum(axis=-1, keepdims=True)
        out[h] = probs @ v[h // group]
    return out.transpose(1, 0, 2).reshape(M, n_heads * hd)
