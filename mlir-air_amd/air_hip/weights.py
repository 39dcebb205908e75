"""AutoAWQ checkpoint loader for the int4 Llama decode path.

Counterpart of load_weights_awq
(programming_examples/llms/llama32_1b_int4/llama32_1b_int4_weights.py:80-238).  The reference
dequantises every linear to bf16 for its prefill path and re-tiles it into per-core decode
buffers; here the W4A16 kernels read the AutoAWQ "gemm" tensors as they are stored, so a
linear stays (qweight int32 [in, out/8], qzeros int32 [in/gs, out/8], scales bf16 [in/gs, out])
and loading is a type check plus one rounding: fp16 scales are rounded to bf16 once
(awq_repacker.py:74-78).  `to_device` moves a loaded model into HBM; `concat_linears` builds the
fused Q|K|V matrix (concatenation along N is a plain concatenation of packed words).

Only local directories are read: there is no network here, and a model id that is not a
directory raises FileNotFoundError instead of trying to download.
"""

import dataclasses
import glob
import os
from typing import List, Optional, Tuple

import numpy as np

from . import awq, bf16

Linear = Tuple[np.ndarray, np.ndarray, np.ndarray]   # (qweight, qzeros, scales bf16 bits)


@dataclasses.dataclass
class LlamaConfig:
    """Model hyperparameters; defaults are Llama-3.2-1B
    (programming_examples/llms/llama32_1b/llama32_1b_weights.py:35-47)."""

    n_layers: int = 16
    emb_dim: int = 2048
    n_heads: int = 32
    head_dim: int = 64
    n_kv_heads: int = 8
    hidden_dim: int = 8192
    vocab_size: int = 128256
    rope_base: float = 500000.0
    rms_eps: float = 1e-5

    @property
    def kv_dim(self):
        return self.n_kv_heads * self.head_dim


# HF AutoAWQ Linear suffix -> field name (llama32_1b_int4_weights.py:58-66)
HF_AWQ_LINEARS = {
    "self_attn.q_proj": "wq",
    "self_attn.k_proj": "wk",
    "self_attn.v_proj": "wv",
    "self_attn.o_proj": "wo",
    "mlp.gate_proj": "w_gate",
    "mlp.up_proj": "w_up",
    "mlp.down_proj": "w_down",
}


@dataclasses.dataclass
class LayerWeights:
    """One transformer layer.  Norm weights are bf16 bit patterns [emb]; every linear is an
    AWQ triple with W[in, out] = y = x @ W orientation."""

    attn_norm: np.ndarray
    ffn_norm: np.ndarray
    wq: Linear
    wk: Linear
    wv: Linear
    wo: Linear
    w_gate: Linear
    w_up: Linear
    w_down: Linear


@dataclasses.dataclass
class LlamaWeights:
    embed_table: np.ndarray      # bf16 bits [vocab, emb]
    layers: List[LayerWeights]
    final_norm: np.ndarray       # bf16 bits [emb]
    lm_head: np.ndarray          # bf16 bits [vocab, emb] (the embedding table when tied)


def resolve_safetensor_files(model_path):
    """All *.safetensors shards of a local checkpoint directory, sorted."""
    if not os.path.isdir(model_path):
        raise FileNotFoundError(
            f"'{model_path}' is not a local directory; downloading checkpoints is not supported here")
    files = sorted(glob.glob(os.path.join(model_path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"No .safetensors files found in {model_path}")
    return files


def _bf16_bits(t):
    """torch tensor (bf16 / fp16 / fp32) -> uint16 bf16 bit patterns, one RNE rounding."""
    import torch

    if t.dtype != torch.bfloat16:
        t = t.to(torch.float32).to(torch.bfloat16)
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _int32(t):
    import torch

    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    return t.contiguous().numpy()


def check_linear(name, qweight, qzeros, scales, group_size):
    K, nb = qweight.shape
    if K % group_size or qzeros.shape != (K // group_size, nb) or scales.shape != (K // group_size, nb * 8):
        raise ValueError(f"{name}: shapes qweight {qweight.shape}, qzeros {qzeros.shape}, scales {scales.shape} "
                         f"are not an AutoAWQ gemm linear with group size {group_size}")


def load_weights_awq(model_name_or_path, config: Optional[LlamaConfig] = None, group_size=awq.GROUP) -> LlamaWeights:
    """Load a local HuggingFace AutoAWQ Llama checkpoint."""
    from safetensors import safe_open

    if config is None:
        config = LlamaConfig()
    files = resolve_safetensor_files(model_name_or_path)
    shard_of = {}   # tensor name -> the shard that holds it
    for path in files:
        with safe_open(path, framework="pt") as f:
            shard_of.update((key, path) for key in f.keys())

    def tensor(key, what="weight"):
        path = shard_of.get(key)
        if path is None:
            hint = "; the directory holds no qweight / qzeros / scales triple under that name, so it was not written by AutoAWQ" if what == "AWQ tensor" else ""
            raise KeyError(f"{what} {key} is in none of the {len(files)} safetensors shard(s){hint}")
        with safe_open(path, framework="pt") as f:
            return f.get_tensor(key)

    embed_table = _bf16_bits(tensor("model.embed_tokens.weight"))
    if embed_table.shape != (config.vocab_size, config.emb_dim):
        raise ValueError(f"embed_table shape mismatch: expected ({config.vocab_size}, {config.emb_dim}), got {embed_table.shape}")

    expect = {
        "wq": (config.emb_dim, config.n_heads * config.head_dim), "wk": (config.emb_dim, config.kv_dim),
        "wv": (config.emb_dim, config.kv_dim), "wo": (config.n_heads * config.head_dim, config.emb_dim),
        "w_gate": (config.emb_dim, config.hidden_dim), "w_up": (config.emb_dim, config.hidden_dim),
        "w_down": (config.hidden_dim, config.emb_dim),
    }
    layers = []
    for i in range(config.n_layers):
        fields = {
            "attn_norm": _bf16_bits(tensor(f"model.layers.{i}.input_layernorm.weight")),
            "ffn_norm": _bf16_bits(tensor(f"model.layers.{i}.post_attention_layernorm.weight")),
        }
        for suffix, field in HF_AWQ_LINEARS.items():
            base = f"model.layers.{i}.{suffix}"
            qw = _int32(tensor(f"{base}.qweight", "AWQ tensor"))
            qz = _int32(tensor(f"{base}.qzeros", "AWQ tensor"))
            sc = _bf16_bits(tensor(f"{base}.scales", "AWQ tensor"))
            check_linear(base, qw, qz, sc, group_size)
            if (qw.shape[0], qw.shape[1] * 8) != expect[field]:
                raise ValueError(f"{base}: [in, out] = {(qw.shape[0], qw.shape[1] * 8)}, config expects {expect[field]}")
            fields[field] = (qw, qz, sc)
        layers.append(LayerWeights(**fields))

    final_norm = _bf16_bits(tensor("model.norm.weight"))
    lm_head = _bf16_bits(tensor("lm_head.weight")) if "lm_head.weight" in shard_of else embed_table
    return LlamaWeights(embed_table=embed_table, layers=layers, final_norm=final_norm, lm_head=lm_head)


def concat_linears(*linears: Linear) -> Linear:
    """Stack AWQ linears that share their input along the output axis (e.g. Q | K | V)."""
    K = linears[0][0].shape[0]
    for qw, _, _ in linears:
        if qw.shape[0] != K:
            raise ValueError("concat_linears: input sizes differ")
    return tuple(np.ascontiguousarray(np.concatenate([l[j] for l in linears], axis=1)) for j in range(3))


def interleaved_gate_up_l1(layer: LayerWeights):
    """The reference's decode layout of the FFN front half: kernel-side arrays with row 2i =
    gate[i], row 2i + 1 = up[i] (llama32_1b_int4_weights.py:173-207)."""
    conv = lambda l: awq.l1_from_awq(l[0], l[1], bf16.from_bits(l[2]))
    return awq.interleave_rows(conv(layer.w_gate), conv(layer.w_up))


def reference_decode_buffers(layer: LayerWeights, group_size=awq.GROUP, m_tile=8, k_chunk=2048, n_cores=8):
    """The per-layer buffers the reference attaches for its decode kernels (`_wq_packed` ...
    `_wgateup_packed`, llama32_1b_int4_weights.py:71-77, 214-216), for interchange with it."""
    out = {}
    for field in ("wq", "wk", "wv", "wo", "w_down"):
        qw, qz, sc = getattr(layer, field)
        a_q, a_s, a_z = awq.l1_from_awq(qw, qz, bf16.from_bits(sc))
        M, K = a_q.shape[0], a_q.shape[1] * 2
        out[f"_{field.replace('w_', 'w')}_packed"] = awq.pack_bo_tiles(a_q, a_s, a_z, M, K, group_size, m_tile,
                                                                    min(k_chunk, K), n_cores, M)
    g_q, g_s, g_z = interleaved_gate_up_l1(layer)
    M, K = g_q.shape[0], g_q.shape[1] * 2
    out["_wgateup_packed"] = awq.pack_bo_tiles(g_q, g_s, g_z, M, K, group_size, m_tile, min(k_chunk, K), n_cores, M)
    return out


def reference_prefill_buffers(layer: LayerWeights, group_size=awq.GROUP, n_tile=16, k_chunk=128):
    """The per-layer dict of packed GEMM buffers the reference's int4 prefill consumes (`layers_packed[i]` of
    load_awq_weights, llama32_1b_int4/awq_pack.py:246-266: wq, wk, wv, wo, w_gate, w_up, w_down, each
    awq_pack_for_npu of the checkpoint tensors), for interchange with it."""
    out = {}
    for field in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
        qw, qz, sc = getattr(layer, field)
        w_q, w_s, w_z = awq.l1_from_awq(qw, qz, bf16.from_bits(sc))
        N, K = w_q.shape[0], w_q.shape[1] * 2
        out[field] = awq.pack_gemm_tiles(w_q, w_s, w_z, K, N, group_size, n_tile, k_chunk)
    return out


def to_device(weights: LlamaWeights, device="cuda"):
    """Copy a loaded model into HBM as torch tensors (bf16 where the host holds bf16 bits)."""
    import torch

    def dev(a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.uint16:
            return torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
        return torch.from_numpy(a).to(device)

    def lin(l):
        return tuple(dev(t) for t in l)

    layers = []
    for lw in weights.layers:
        d = {f.name: getattr(lw, f.name) for f in dataclasses.fields(lw)}
        layers.append(LayerWeights(**{k: (lin(v) if isinstance(v, tuple) else dev(v)) for k, v in d.items()}))
    embed = dev(weights.embed_table)
    lm_head = embed if weights.lm_head is weights.embed_table else dev(weights.lm_head)
    return LlamaWeights(embed_table=embed, layers=layers, final_norm=dev(weights.final_norm), lm_head=lm_head)
