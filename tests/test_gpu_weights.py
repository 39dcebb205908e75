"""A checkpoint on disk through the whole decode path on the GPU: a synthetic AutoAWQ safetensors directory (two
shards, fp16 scales, the reference's tensor names) -> load_weights_awq -> prepare_layer -> run_decode_block, against
the oracle's decode block fed the checkpoint's own tensors (load_weights_awq,
programming_examples/llms/llama32_1b_int4/llama32_1b_int4_weights.py:80-238; fp16 -> bf16 scale rounding,
awq_repacker.py:74-78; run_decode_block, llama32_1b_int4_decode.py:176-313).  No AWQ checkpoint exists offline, so
the directory is written by the test."""
import numpy as np
import pytest
import torch

from helpers import bf16_ulp
from oracle import awq as oawq, decode as odec, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits
from test_weights_cpu import CFG, _write_checkpoint

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def test_loaded_checkpoint_decodes_like_the_oracle(tmp_path):
    from air_hip import decode, weights

    print("checkpoint -> loader -> prepare_layer -> decode blocks", flush=True)
    src = _write_checkpoint(str(tmp_path / "ckpt"), tied=True, seed=11)
    # projections scaled down so that activations stay O(1) through two blocks: rewrite the scales in the files'
    # own dtype (fp16) before loading, so the loader still does the fp16 -> bf16 rounding
    from safetensors.torch import load_file, save_file
    import glob, os
    for f in glob.glob(os.path.join(str(tmp_path / "ckpt"), "*.safetensors")):
        sh = load_file(f)
        for k in sh:
            if k.endswith(".scales"):
                sh[k] = (sh[k].float() * 0.25).to(torch.float16)
                src[k] = sh[k]
        save_file(sh, f)
    w = weights.load_weights_awq(str(tmp_path / "ckpt"), CFG)
    layers = [decode.prepare_layer(lw) for lw in w.layers]

    # the oracle reads the checkpoint tensors directly: int32 words as stored, fp16 scales rounded to bf16 once
    def l1(i):
        names = {"wq": "self_attn.q_proj", "wk": "self_attn.k_proj", "wv": "self_attn.v_proj", "wo": "self_attn.o_proj",
                 "w_gate": "mlp.gate_proj", "w_up": "mlp.up_proj", "w_down": "mlp.down_proj"}
        out = {}
        for field, hf in names.items():
            base = f"model.layers.{i}.{hf}"
            sc = f32_to_bf16_bits(src[base + ".scales"].numpy().astype(np.float32))
            out[field] = oawq.repack_hf_awq_linear(src[base + ".qweight"].numpy(), src[base + ".qzeros"].numpy(), sc, 128)
        out["attn_norm"] = src[f"model.layers.{i}.input_layernorm.weight"].view(torch.int16).numpy().view(np.uint16)
        out["ffn_norm"] = src[f"model.layers.{i}.post_attention_layernorm.weight"].view(torch.int16).numpy().view(np.uint16)
        return out

    max_seq = 8
    lut_bits = odec.generate_rope_lut(CFG.head_dim, CFG.rope_base, max_seq)
    lut = decode.generate_rope_lut(CFG, max_seq)
    cache = decode.new_kv_cache(CFG, max_seq)
    ref_cache = [(np.zeros((CFG.n_kv_heads, max_seq, CFG.head_dim), np.uint16), np.zeros((CFG.n_kv_heads, max_seq, CFG.head_dim), np.uint16))
                 for _ in range(CFG.n_layers)]
    rng = np.random.default_rng(5)
    for pos in range(3):
        x = w.embed_table[int(rng.integers(0, CFG.vocab_size))]
        xd = dev(x)
        for i in range(CFG.n_layers):
            (kc, vc), (kr, vr) = cache[i], ref_cache[i]
            y = decode.run_decode_block(xd, layers[i], CFG, kc, vc, pos, lut)
            torch.cuda.synchronize()
            want = odec.decode_block_reference(x, l1(i), kr, vr, pos, lut_bits, CFG.n_heads, CFG.n_kv_heads, CFG.head_dim)
            got_f, want_f = bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(want)
            assert oref.check_outputs(got_f, want_f, rtol=0.2, atol=2.0, min_correlation=0.99), (pos, i)
            assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), (pos, i, np.max(np.abs(got_f - want_f)))
            kd = np.abs(bf16_bits_to_f32(bits(kc)[:, pos]) - bf16_bits_to_f32(kr[:, pos]))
            assert np.all(kd <= 2 * bf16_ulp(bf16_bits_to_f32(kr[:, pos])) + 2e-2), kd.max()
            # both sides continue from the oracle's values
            kc[:, pos] = dev(kr[:, pos])
            vc[:, pos] = dev(vr[:, pos])
            x, xd = want, dev(want)
