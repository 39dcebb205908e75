"""One int4 decode step on the GPU: the counterpart of run_decode_block
(programming_examples/llms/llama32_1b_int4/llama32_1b_int4_decode.py:176-313).

The reference issues two NPU calls per layer (rms_qkv_int4_rope: 6 launches; o_gemv_ffn_int4:
3 launches) with the KV-cache update and the attention on the host CPU in between.  Here a layer
is five kernel launches, all on the device:

  1. RMSNorm + fused Q|K|V int4 GEMV (one matrix, concatenated along the output axis)
  2. RoPE(Q, K) + cache append + grouped-query attention (+ 3. the chunk combine for long contexts, unless the O
     projection can merge the chunks itself)
  4-6. O projection + residual, RMSNorm + gate/up + SwiGLU, down projection + residual
"""

import dataclasses

import numpy as np
import torch

from . import ops, weights as wmod


def generate_rope_lut(config, seq_len=2048, device="cuda"):
    """bf16 [seq_len, head_dim]: cos(pos * f_i) for i < head_dim / 2, then sin(pos * f_i), with
    f_i = rope_base^(-2i / head_dim) evaluated in float64 and rounded once
    (programming_examples/llms/llama32_1b/llama32_1b_weights.py:395-444)."""
    hd = config.head_dim
    inv_freq = 1.0 / (config.rope_base ** (np.arange(0, hd, 2, dtype=np.float64) / hd))
    angles = np.outer(np.arange(seq_len, dtype=np.float64), inv_freq)
    lut = np.concatenate([np.cos(angles), np.sin(angles)], axis=1).astype(np.float32)
    return torch.from_numpy(lut).to(torch.bfloat16).to(device)


@dataclasses.dataclass
class DecodeLayer:
    """Device tensors of one layer in the form the kernels read."""

    attn_norm: torch.Tensor
    ffn_norm: torch.Tensor
    wqkv: tuple       # fused (qweight, qzeros, scales), N = (n_heads + 2 n_kv) * head_dim
    wo: tuple
    w_gate: tuple
    w_up: tuple
    w_down: tuple
    codec: str = "awq"   # "awq": triples are (qweight, qzeros, scales); "q4nx": (qweight, scales, mins) from q4nx_repack
    # The same five matrices in stream order (ops.StreamWeight; Q4NX order for that codec), which the decode kernels
    # and the prompt pass read.  None: an AWQ layer whose widths the stream order does not take runs on the triples.
    stream: dict = None

    def with_stream(self, keep_triples=False):
        """Re-pack the layer's matrices into stream order on the GPU (once, at load time).  A layer with a matrix the
        stream order does not take (N % 16 != 0) keeps its triples and runs the checkpoint-layout kernels.  Unless
        `keep_triples`, the triples are dropped once nothing reads them any more, i.e. when the prompt pass also takes
        the stream-order copies (Q4NX layers: always), so that the weights are held once."""
        names = ("wqkv", "wo", "w_gate", "w_up", "w_down")
        if self.stream is None:
            if self.codec == "awq" and any(getattr(self, n)[0].shape[1] * 8 % 16 for n in names):
                return self
            repack = ops.repack_stream if self.codec == "awq" else ops.q4nx_repack_stream
            self.stream = {name: repack(*getattr(self, name)) for name in names}
        if not keep_triples and (self.codec != "awq" or _stream_covers_prefill(self.stream)):
            self.wqkv = self.wo = self.w_gate = self.w_up = self.w_down = None
        return self


def _stream_covers_prefill(sw):
    """Whether the prompt pass runs on these stream-order copies (run_prefill_layer): input lengths in whole pairs of
    groups, widths in whole 64-column tiles, attention output as wide as the embedding."""
    E, H, nq, nqkv = sw["w_gate"].K, sw["w_gate"].N, sw["wo"].K, sw["wqkv"].N
    return E % 256 == 0 and H % 256 == 0 and nq == E and nqkv % 64 == 0


def prepare_layer_q4nx(blocks, attn_norm, ffn_norm, config, mode=0, device="cuda") -> DecodeLayer:
    """A Q4NX / Q4_0 layer -> DecodeLayer.  `blocks` maps q, k, v, o, gate, up, down to the tensor's
    blocks (uint8 [n_blocks, 5120], numpy or torch) in (row-block, col-block) order as a model.q4nx
    bundle stores them; Q, K, V are fused by concatenating their blocks (whole row-blocks of the output
    axis), and every matrix is re-packed on the GPU, in one pass, into the Q4NX stream order that the decode kernels
    and the prompt pass read (as the reference re-packs the blocks once into its cascade order, proj_qmm_pack.py:61-140).
    Norm weights are bf16 bit patterns or tensors."""
    E, H = config.emb_dim, config.hidden_dim
    nq, nkv = config.n_heads * config.head_dim, config.kv_dim

    def dev_blocks(b):
        t = b if isinstance(b, torch.Tensor) else torch.from_numpy(np.ascontiguousarray(np.asarray(b).view(np.uint8)))
        return t.to(device).reshape(-1, 5120)

    def dev_vec(a):
        if isinstance(a, torch.Tensor):
            return a.to(device)
        return torch.from_numpy(np.ascontiguousarray(np.asarray(a).view(np.int16))).to(device).view(torch.bfloat16)

    def repack(t, M, K):
        return ops.q4nx_blocks_to_stream(t.contiguous(), M, K, mode)

    qkv = torch.cat([dev_blocks(blocks[n]) for n in ("q", "k", "v")], dim=0)
    stream = {"wqkv": repack(qkv, nq + 2 * nkv, E), "wo": repack(dev_blocks(blocks["o"]), E, nq),
              "w_gate": repack(dev_blocks(blocks["gate"]), H, E), "w_up": repack(dev_blocks(blocks["up"]), H, E),
              "w_down": repack(dev_blocks(blocks["down"]), E, H)}
    return DecodeLayer(attn_norm=dev_vec(attn_norm), ffn_norm=dev_vec(ffn_norm), wqkv=None, wo=None, w_gate=None, w_up=None,
                       w_down=None, codec="q4nx", stream=stream)


def prepare_layer(layer: wmod.LayerWeights, device="cuda", stream_order=True, keep_triples=False) -> DecodeLayer:
    """Host LayerWeights (numpy) -> DecodeLayer: Q, K, V concatenated, everything in HBM, and (stream_order) every
    matrix re-packed into the decode kernels' stream order, the counterpart of the packed decode buffers the
    reference attaches per layer at load time (llama32_1b_int4_weights.py:163-216).  stream_order=False leaves the
    AutoAWQ triples for the checkpoint-layout kernels; keep_triples keeps them beside the re-pack."""
    def dev(a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.uint16:
            return torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
        return torch.from_numpy(a).to(device)

    lin = lambda l: tuple(dev(t) for t in l)
    out = DecodeLayer(attn_norm=dev(layer.attn_norm), ffn_norm=dev(layer.ffn_norm),
                      wqkv=lin(wmod.concat_linears(layer.wq, layer.wk, layer.wv)), wo=lin(layer.wo),
                      w_gate=lin(layer.w_gate), w_up=lin(layer.w_up), w_down=lin(layer.w_down))
    return out.with_stream(keep_triples) if stream_order else out


def new_kv_cache(config, max_seq, device="cuda"):
    """Per-layer caches [n_kv_heads, max_seq, head_dim] bf16 (the reference's layout)."""
    shape = (config.n_kv_heads, max_seq, config.head_dim)
    return [(torch.zeros(shape, dtype=torch.bfloat16, device=device), torch.zeros(shape, dtype=torch.bfloat16, device=device))
            for _ in range(config.n_layers)]


def run_decode_block(x, layer: DecodeLayer, config, k_cache_layer, v_cache_layer, current_pos, rope_lut, x_sumsq=None,
                     return_sumsq=False):
    """One transformer block for one decode token; x bf16 [emb] -> bf16 [emb].  The caches are
    updated in place at current_pos.  x_sumsq / return_sumsq chain the sum of squares of the block's output into
    the next block's RMSNorm (AWQ layers): with return_sumsq the result is (y, sumsq or None)."""
    q4nx = layer.codec == "q4nx"
    if layer.stream is not None and q4nx:   # Q4NX order: the same whole-K launches, attention as its own call
        sw = layer.stream
        qkv = ops.q4nx_rms_gemv_stream(x, layer.attn_norm, sw["wqkv"], eps=config.rms_eps, x_sumsq=x_sumsq)
        attn_out = ops.decode_attention(qkv, rope_lut[current_pos], k_cache_layer, v_cache_layer, current_pos, config.n_heads)
        return ops.q4nx_o_gemv_ffn_stream(attn_out, x, layer.ffn_norm, sw["wo"], sw["w_gate"], sw["w_up"], sw["w_down"],
                                          eps=config.rms_eps, return_sumsq=return_sumsq)
    if layer.stream is not None:   # stream-order weights: stateless whole-K launches, sums of squares per 16 columns
        sw = layer.stream
        qkv = ops.w4a16_rms_gemv_stream(x, layer.attn_norm, sw["wqkv"], eps=config.rms_eps, x_sumsq=x_sumsq)
        return ops.decode_attn_o_gemv_ffn_stream(qkv, rope_lut[current_pos], k_cache_layer, v_cache_layer, current_pos,
                                                 config.n_heads, x, layer.ffn_norm, sw["wo"], sw["w_gate"], sw["w_up"],
                                                 sw["w_down"], eps=config.rms_eps, return_sumsq=return_sumsq)
    if q4nx:
        raise ValueError("a Q4NX layer runs on its stream-order re-pack (prepare_layer_q4nx / DecodeLayer.with_stream)")
    # AutoAWQ triples (widths the stream order does not take, or a layer prepared with stream_order=False): attention +
    # block as one call, the O projection merges the attention's chunk partials where it can
    qkv = ops.w4a16_rms_gemv(x, layer.attn_norm, *layer.wqkv, eps=config.rms_eps, x_sumsq=x_sumsq)
    return ops.decode_attn_o_gemv_ffn(qkv, rope_lut[current_pos], k_cache_layer, v_cache_layer, current_pos, config.n_heads,
                                      x, layer.ffn_norm, layer.wo, layer.w_gate, layer.w_up, layer.w_down, eps=config.rms_eps,
                                      return_sumsq=return_sumsq)


def decode_token(token_id, layers, embed_table, final_norm, lm_head, config, kv_cache, current_pos, rope_lut,
                 return_argmax=False):
    """Full model step: embedding row -> blocks -> final RMSNorm + bf16 lm_head GEMV (+ argmax) in one
    kernel call (run_npu_decode_step, llama32_1b_int4_inference.py:429-486).  Returns the logits as
    fp32 [vocab], like the reference, and with return_argmax also the greedy token as a device
    int32 tensor [1] (no host synchronisation here)."""
    x = embed_table[token_id].contiguous()
    sumsq = None   # every block leaves the sum of squares of its output for the next block's norm
    for layer, (kc, vc) in zip(layers, kv_cache):
        x, sumsq = run_decode_block(x, layer, config, kc, vc, current_pos, rope_lut, x_sumsq=sumsq, return_sumsq=True)
    logits, best = ops.lm_head(x, lm_head, norm_weight=final_norm, eps=config.rms_eps)
    return (logits.float(), best) if return_argmax else logits.float()


def decode_greedy(token, n_tokens, layers, embed_table, final_norm, lm_head, config, kv_cache, start_pos, rope_lut):
    """Greedy decode loop of `generate` (llama32_1b_int4_inference.py:494-560) with nothing returning
    to the host between tokens: `token` is a device int32 tensor [1] (the token at position
    start_pos), each step's argmax feeds the next embedding lookup on the device.  Returns the
    n_tokens generated ids as a device int32 tensor; the caller looks for an end-of-sequence id
    afterwards (the reference stops at it, so later entries are to be dropped)."""
    out = torch.empty((n_tokens,), dtype=torch.int32, device=embed_table.device)
    tok = token.to(torch.int32).reshape(1)
    for i in range(n_tokens):
        x = embed_table.index_select(0, tok).reshape(-1)
        sumsq = None
        for layer, (kc, vc) in zip(layers, kv_cache):
            x, sumsq = run_decode_block(x, layer, config, kc, vc, start_pos + i, rope_lut, x_sumsq=sumsq, return_sumsq=True)
        tok = out[i:i + 1]   # the argmax lands in the ids buffer; the next embedding lookup reads it from there
        ops.lm_head(x, lm_head, norm_weight=final_norm, eps=config.rms_eps, argmax_out=tok)
    return out


def run_prefill_layer(x, layer: DecodeLayer, config, k_cache_layer, v_cache_layer, rope_lut):
    """One transformer block over the M prompt tokens at positions 0..M-1 (_run_layer_int4,
    programming_examples/llms/llama32_1b_int4/llama32_1b_int4_prefill.py:241-390): RMSNorm + fused Q|K|V GEMM +
    RoPE, causal attention, O projection + FFN block; x bf16 [M, emb] -> bf16 [M, emb].  The roped K and V
    rows are written to the caches [n_kv_heads, max_seq, head_dim] at positions 0..M-1, where the decode
    steps that follow expect them."""
    M = x.shape[0]
    nh, nkv, hd = config.n_heads, config.n_kv_heads, config.head_dim
    # the stream-order copies where the layer has them and the tiled stream-order GEMM takes every matrix
    sw = layer.stream if layer.stream is not None and _stream_covers_prefill(layer.stream) else None
    if layer.codec != "awq" and sw is None:
        # (the reference prefills its Q4NX models as dense bf16 GEMMs on dequantised weights; the tiled kernel multiplies
        # the same bf16 values from the Q4NX order and has no checkpoint-layout twin)
        raise ValueError("a Q4NX layer is prefilled from its stream-order re-pack: E, H multiples of 256, widths of 64")
    if sw is not None:
        qkv = ops.prefill_rms_qkv_rope_stream(x, layer.attn_norm, sw["wqkv"], rope_lut, 0, nh, nkv, hd, eps=config.rms_eps,
                                              codec=layer.codec)
    else:
        qkv = ops.prefill_rms_qkv_rope(x, layer.attn_norm, layer.wqkv, rope_lut, 0, nh, nkv, hd, eps=config.rms_eps)
    nq, nk = nh * hd, nkv * hd
    k_cache_layer[:, :M].copy_(qkv[:, nq:nq + nk].reshape(M, nkv, hd).transpose(0, 1))
    v_cache_layer[:, :M].copy_(qkv[:, nq + nk:].reshape(M, nkv, hd).transpose(0, 1))
    attn_out = ops.prefill_attention(qkv, nh, nkv, hd)
    if sw is not None:
        return ops.prefill_o_ffn_stream(attn_out, x, layer.ffn_norm, sw["wo"], sw["w_gate"], sw["w_up"], sw["w_down"], eps=config.rms_eps,
                                        codec=layer.codec)
    return ops.prefill_o_ffn(attn_out, x, layer.ffn_norm, layer.wo, layer.w_gate, layer.w_up, layer.w_down, eps=config.rms_eps)


def prefill(token_ids, layers, embed_table, final_norm, lm_head, config, kv_cache, rope_lut):
    """Prompt pass (run_npu_prefill, llama32_1b_int4_inference.py:335-427): all prompt tokens through every
    layer at once, KV caches filled for positions 0..M-1, then the decode tail on the last row only.
    token_ids: device integer tensor [M].  Returns (logits fp32 [vocab] of the last position, greedy next
    token as a device int32 tensor [1])."""
    x = embed_table.index_select(0, token_ids.to(torch.int32)).contiguous()
    for layer, (kc, vc) in zip(layers, kv_cache):
        x = run_prefill_layer(x, layer, config, kc, vc, rope_lut)
    logits, best = ops.lm_head(x[-1].contiguous(), lm_head, norm_weight=final_norm, eps=config.rms_eps)
    return logits.float(), best


def generate(prompt_tokens, layers, embed_table, final_norm, lm_head, config, rope_lut, n_tokens=10,
             eos_token_ids=(128001, 128009), on_token=None):
    """Prompt pass + greedy decode (generate, programming_examples/llms/llama32_1b_int4/llama32_1b_int4_inference.py:494-575):
    returns [first token predicted by the prompt pass] + the tokens decoded after it, at most n_tokens of them,
    ending with the first end-of-sequence id if one is produced.  prompt_tokens: a sequence of ints.

    Without `on_token` the whole decode loop runs on the device (decode_greedy) and the ids come back once; tokens
    after an end-of-sequence id are computed and dropped.  With `on_token(token_id)` every token is brought to the
    host as it is produced (the reference's streaming mode) and the loop stops at an end-of-sequence id."""
    seq_len = len(prompt_tokens)
    max_seq = seq_len + n_tokens
    if rope_lut.shape[0] < max_seq:
        raise ValueError(f"the RoPE table has {rope_lut.shape[0]} rows, the run needs {max_seq}")
    kv_cache = new_kv_cache(config, max_seq, device=embed_table.device)
    ids = torch.as_tensor(list(prompt_tokens), dtype=torch.int32, device=embed_table.device)
    _, first = prefill(ids, layers, embed_table, final_norm, lm_head, config, kv_cache, rope_lut)
    eos = set(int(t) for t in eos_token_ids)
    if on_token is None:
        rest = decode_greedy(first, n_tokens, layers, embed_table, final_norm, lm_head, config, kv_cache, seq_len, rope_lut)
        ops.check_health()
        out = [int(first.item())] + [int(t) for t in rest.cpu().tolist()]
        for i in range(1, len(out)):
            if out[i] in eos:
                return out[:i + 1]
        return out
    tok = int(first.item())
    out = [tok]
    on_token(tok)
    for i in range(n_tokens):
        _, best = decode_token(tok, layers, embed_table, final_norm, lm_head, config, kv_cache, seq_len + i, rope_lut,
                               return_argmax=True)
        ops.check_health()
        tok = int(best.item())
        out.append(tok)
        on_token(tok)
        if tok in eos:
            break
    return out
