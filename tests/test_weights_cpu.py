"""Checkpoint loader and the reference's tiled decode-buffer layout (CPU only)."""
import os

import numpy as np
import pytest
import torch

from air_hip import awq, bf16, weights
from oracle import awq as oawq
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def _l1(M, K, gs, seed):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    a_q = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    a_s = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // gs, M)).astype(np.float32))
    a_z = rng.integers(0, 16, size=(K // gs, M), dtype=np.uint8)
    return a_q, a_s, a_z


@pytest.mark.parametrize("mpl", [16, 32])
def test_bo_tiles_match_the_loop_restatement_and_invert(mpl):
    M, K, GS, M_TILE, K_CHUNK, N_CORES = 32, 512, 128, 4, 256, 2
    a_q, a_s, a_z = _l1(M, K, GS, 1)
    got = awq.pack_bo_tiles(a_q, bf16.from_bits(a_s), a_z, M, K, GS, M_TILE, K_CHUNK, N_CORES, mpl)
    want = oawq.pack_inputs_loop(a_q, a_s, a_z, M, K, GS, M_TILE, K_CHUNK, N_CORES, mpl)
    assert got.shape == want.shape == (M // M_TILE * (K // K_CHUNK), 4 * 128 + 2 * 4 * 2 + 2 * 4)
    assert np.array_equal(got, want)
    b_q, b_s, b_z = awq.unpack_bo_tiles(got, M, K, GS, M_TILE, K_CHUNK, N_CORES, mpl)
    assert np.array_equal(b_q, a_q) and np.array_equal(bf16.bits_of(b_s), a_s) and np.array_equal(b_z, a_z)


def test_bo_tile_byte_offsets_by_hand():
    # one element followed by hand: row 13, k = 300 (odd k -> high nibble of byte 150), group 2
    M, K, GS, M_TILE, K_CHUNK, N_CORES = 16, 512, 128, 8, 256, 2
    a_q = np.zeros((M, K // 2), np.uint8)
    a_s = np.zeros((K // GS, M), np.uint16)
    a_z = np.zeros((K // GS, M), np.uint8)
    a_q[13, 150] = 0xA0
    a_s[2, 13] = 0x3C12
    a_z[2, 13] = 9
    for packed in (awq.pack_bo_tiles(a_q, bf16.from_bits(a_s), a_z, M, K, GS, M_TILE, K_CHUNK, N_CORES),
                   oawq.pack_inputs_loop(a_q, a_s, a_z, M, K, GS, M_TILE, K_CHUNK, N_CORES, M)):
        # row block 1 (rows 8..15), K chunk 1 (k 256..511) -> tile 1 * 2 + 1 = 3; row 5 of the tile;
        # byte 150 - 128 = 22 of the chunk; group 2 is group 0 of the chunk
        tile = packed[3]
        q_bytes, s_bytes = 8 * 128, 2 * 8 * 2
        assert tile[5 * 128 + 22] == 0xA0
        assert tile[q_bytes + 2 * (0 * 8 + 5)] == 0x12 and tile[q_bytes + 2 * (0 * 8 + 5) + 1] == 0x3C
        assert tile[q_bytes + s_bytes + 0 * 8 + 5] == 9
        assert int(packed.astype(np.int64).sum()) == 0xA0 + 0x12 + 0x3C + 9


def test_bo_tiles_reject_a_tiling_that_does_not_divide():
    a_q, a_s, a_z = _l1(24, 256, 128, 2)
    with pytest.raises(ValueError):
        awq.pack_bo_tiles(a_q, bf16.from_bits(a_s), a_z, 24, 256, 128, 8, 256, 2)
    with pytest.raises(ValueError):
        awq.unpack_bo_tiles(np.zeros(10, np.uint8), 32, 256, 128, 8, 256, 2)


CFG = weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64, n_kv_heads=2, hidden_dim=512, vocab_size=64)


def _write_checkpoint(path, tied, seed=0, drop=None):
    from safetensors.torch import save_file

    g = torch.Generator().manual_seed(seed)
    shards = [{}, {}]

    def put(i, key, t):
        if key != drop:
            shards[i][key] = t.contiguous()

    put(0, "model.embed_tokens.weight", torch.randn((CFG.vocab_size, CFG.emb_dim), generator=g).to(torch.bfloat16))
    shapes = {"self_attn.q_proj": (256, 256), "self_attn.k_proj": (256, 128), "self_attn.v_proj": (256, 128),
              "self_attn.o_proj": (256, 256), "mlp.gate_proj": (256, 512), "mlp.up_proj": (256, 512),
              "mlp.down_proj": (512, 256)}
    for i in range(CFG.n_layers):
        put(i % 2, f"model.layers.{i}.input_layernorm.weight", (torch.randn(256, generator=g) * 0.1 + 1).to(torch.bfloat16))
        put(i % 2, f"model.layers.{i}.post_attention_layernorm.weight", (torch.randn(256, generator=g) * 0.1 + 1).to(torch.bfloat16))
        for name, (K, N) in shapes.items():
            base = f"model.layers.{i}.{name}"
            put(i % 2, base + ".qweight", torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, generator=g))
            put((i + 1) % 2, base + ".qzeros", torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, generator=g))
            put(i % 2, base + ".scales", (torch.rand((K // 128, N), generator=g) * 0.015 + 0.005).to(torch.float16))
    put(1, "model.norm.weight", torch.ones(256, dtype=torch.bfloat16))
    if not tied:
        put(1, "lm_head.weight", torch.randn((CFG.vocab_size, CFG.emb_dim), generator=g).to(torch.bfloat16))
    os.makedirs(path, exist_ok=True)
    for j, sh in enumerate(shards):
        save_file(sh, os.path.join(path, f"model-{j:05d}-of-00002.safetensors"))
    return {k: v for sh in shards for k, v in sh.items()}


def test_loader_reads_an_autoawq_checkpoint(tmp_path):
    src = _write_checkpoint(str(tmp_path / "ckpt"), tied=False)
    w = weights.load_weights_awq(str(tmp_path / "ckpt"), CFG)
    assert len(w.layers) == 2 and w.lm_head is not w.embed_table
    assert np.array_equal(w.embed_table, src["model.embed_tokens.weight"].view(torch.int16).numpy().view(np.uint16))
    qw, qz, sc = w.layers[1].w_down
    assert qw.dtype == np.int32 and qw.shape == (512, 32) and qz.shape == (4, 32) and sc.shape == (4, 256)
    assert np.array_equal(qw, src["model.layers.1.mlp.down_proj.qweight"].numpy())
    assert np.array_equal(qz, src["model.layers.1.mlp.down_proj.qzeros"].numpy())
    # fp16 scales are rounded to bf16 once, to nearest even
    s16 = src["model.layers.1.mlp.down_proj.scales"].numpy().astype(np.float32)
    assert np.array_equal(sc, f32_to_bf16_bits(s16))
    assert np.array_equal(w.layers[0].attn_norm,
                          src["model.layers.0.input_layernorm.weight"].view(torch.int16).numpy().view(np.uint16))
    # the loaded triple dequantises like the checkpoint's tensors
    want = oawq.dequant_to_bf16(qw, qz, f32_to_bf16_bits(s16), 128)
    assert np.array_equal(oawq.dequant_to_bf16(*w.layers[1].w_down, 128), want)


def test_loader_tied_embeddings_and_errors(tmp_path):
    _write_checkpoint(str(tmp_path / "tied"), tied=True)
    w = weights.load_weights_awq(str(tmp_path / "tied"), CFG)
    assert w.lm_head is w.embed_table
    _write_checkpoint(str(tmp_path / "broken"), tied=True, drop="model.layers.1.mlp.up_proj.qzeros")
    with pytest.raises(KeyError, match="AutoAWQ"):
        weights.load_weights_awq(str(tmp_path / "broken"), CFG)
    with pytest.raises(FileNotFoundError):
        weights.load_weights_awq("amd/Llama-3.2-1B-Instruct-awq-uint4-asym-g128-bf16-lmhead", CFG)
    os.makedirs(tmp_path / "empty")
    with pytest.raises(FileNotFoundError):
        weights.load_weights_awq(str(tmp_path / "empty"), CFG)
    with pytest.raises(ValueError, match="config expects"):
        weights.load_weights_awq(str(tmp_path / "tied"), weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64,
                                                                           n_kv_heads=4, hidden_dim=512, vocab_size=64))


def test_concat_and_reference_decode_buffers(tmp_path):
    _write_checkpoint(str(tmp_path / "c"), tied=True, seed=3)
    layer = weights.load_weights_awq(str(tmp_path / "c"), CFG).layers[0]
    qkv = weights.concat_linears(layer.wq, layer.wk, layer.wv)
    assert qkv[0].shape == (256, 64) and qkv[2].shape == (2, 512)
    parts = [oawq.dequant_to_bf16(*l, 128) for l in (layer.wq, layer.wk, layer.wv)]
    assert np.array_equal(oawq.dequant_to_bf16(*qkv, 128), np.concatenate(parts, axis=1))
    bufs = weights.reference_decode_buffers(layer, k_chunk=256, n_cores=2)
    assert sorted(bufs) == ["_wdown_packed", "_wgateup_packed", "_wk_packed", "_wo_packed", "_wq_packed", "_wv_packed"]
    # a reference-layout buffer converts back to this backend's tensors
    a = awq.unpack_bo_tiles(bufs["_wdown_packed"], 256, 512, 128, 8, 256, 2)
    back = awq.awq_from_l1(*a)
    assert np.array_equal(back[0], layer.w_down[0]) and np.array_equal(back[1], layer.w_down[1])
    assert np.array_equal(bf16.bits_of(back[2]), layer.w_down[2])
    # gate/up buffer: row 2i = gate[i], 2i + 1 = up[i]
    g = awq.unpack_bo_tiles(bufs["_wgateup_packed"], 1024, 256, 128, 8, 256, 2)
    gate, up = awq.deinterleave_rows(*g)
    assert np.array_equal(awq.awq_from_l1(*gate)[0], layer.w_gate[0]) and np.array_equal(awq.awq_from_l1(*up)[0], layer.w_up[0])


def test_gemm_tiles_match_the_loop_restatement_invert_and_follow_an_element_by_hand():
    K, N, GS, N_TILE, K_CHUNK = 512, 48, 128, 16, 256
    w_q, w_s, w_z = _l1(N, K, GS, 11)
    got = awq.pack_gemm_tiles(w_q, bf16.from_bits(w_s), w_z, K, N, GS, N_TILE, K_CHUNK)
    want = oawq.pack_inputs_gemm_loop(w_q, w_s, w_z, K, N, GS, N_TILE, K_CHUNK)
    assert got.shape == want.shape == (3, 2, 16 * 128 + 2 * 16 * 2 + 2 * 16)
    assert np.array_equal(got, want)
    b_q, b_s, b_z = awq.unpack_gemm_tiles(got, K, N, GS, N_TILE, K_CHUNK)
    assert np.array_equal(b_q, w_q) and np.array_equal(bf16.bits_of(b_s), w_s) and np.array_equal(b_z, w_z)
    # one element by hand: output column 37, k = 301 (high nibble of byte 150), group 2
    z_q, z_s, z_z = np.zeros_like(w_q), np.zeros_like(w_s), np.zeros_like(w_z)
    z_q[37, 150], z_s[2, 37], z_z[2, 37] = 0xB0, 0x3D34, 6
    for packed in (awq.pack_gemm_tiles(z_q, bf16.from_bits(z_s), z_z, K, N, GS, N_TILE, K_CHUNK),
                   oawq.pack_inputs_gemm_loop(z_q, z_s, z_z, K, N, GS, N_TILE, K_CHUNK)):
        tile = packed[2, 1]            # columns 32..47, k 256..511; row 5 of the tile, byte 22 and group 0 of the chunk
        q_bytes, s_bytes = 16 * 128, 2 * 16 * 2
        assert tile[5 * 128 + 22] == 0xB0 and tile[q_bytes + 2 * 5] == 0x34 and tile[q_bytes + 2 * 5 + 1] == 0x3D
        assert tile[q_bytes + s_bytes + 5] == 6 and int(packed.astype(np.int64).sum()) == 0xB0 + 0x34 + 0x3D + 6


def test_awq_tensors_to_gemm_tiles_is_the_reference_prefill_packing():
    """awq_pack_for_npu (awq_pack.py:112-146): unpack the AutoAWQ words, transpose to output-major, pair
    k-neighbours into bytes, tile.  Restated step by step with the oracle's unpacker."""
    K, N, GS = 256, 64, 128
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(0, 16, size=(K // GS, N), dtype=np.uint8)
    sc = f32_to_bf16_bits(rng.uniform(0.005, 0.02, size=(K // GS, N)).astype(np.float32))
    qw, qz = oawq.pack_awq_int32(q), oawq.pack_awq_int32(z)
    layer = weights.LayerWeights(attn_norm=None, ffn_norm=None, **{f: (qw, qz, sc) for f in
                                 ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")})
    got = weights.reference_prefill_buffers(layer, n_tile=16, k_chunk=128)["w_up"]
    w_nk = np.ascontiguousarray(oawq.unpack_awq_int32(qw).T)
    w_q = (w_nk[:, 0::2] | (w_nk[:, 1::2] << 4)).astype(np.uint8)
    want = oawq.pack_inputs_gemm_loop(w_q, sc, oawq.unpack_awq_int32(qz), K, N, GS, 16, 128)
    assert np.array_equal(got, want)


def test_dequant_1d_tile_form_offsets_and_round_trip():
    """The 1-D dequant example's buffer (dequant_awq.py:59-69, 259-278).  Sizes from the formula by hand: n = 1024,
    gs = 128, herd_n = 4 -> 256 elements per tile = 128 Q bytes + 2 groups x 2 S bytes + 2 Z bytes = 134 -> 136.  An
    element followed to its byte: element 777 = tile 3, offset 9 -> byte 4 (high nibble); its group 6 = tile 3, local
    group 0 -> S at bytes 128..129, Z at byte 132."""
    from air_hip import awq, bf16
    from oracle import awq as oawq

    assert awq.packed_tile_bytes_1d(256, 128) == (128, 4, 2, 136)
    assert awq.packed_tile_bytes_1d(128, 128) == (64, 2, 1, 68)        # 67 -> 68
    assert awq.packed_tile_bytes_1d(512, 64) == (256, 16, 8, 280)
    rng = np.random.default_rng(3)
    n, gs, herd_n = 1024, 128, 4
    q = rng.integers(0, 16, n).astype(np.uint8)
    z = rng.integers(0, 16, n // gs).astype(np.uint8)
    s = rng.integers(0, 65536, n // gs).astype(np.uint16)
    packed = awq.pack_inputs_1d(q, bf16.from_bits(s), z, n, gs, herd_n)
    assert packed.shape == (4, 136) and packed.dtype == np.uint8
    assert packed[3, 4] >> 4 == q[777] and packed[3, 4] & 0xF == q[776]
    assert int(packed[3, 128]) | (int(packed[3, 129]) << 8) == s[6] and packed[3, 132] == z[6]
    assert int(packed[3, 130]) | (int(packed[3, 131]) << 8) == s[7] and packed[3, 133] == z[7]
    assert not packed[:, 134:].any()                                    # padding
    assert np.array_equal(packed, oawq.pack_inputs_1d_loop(q, s, z, n, gs, herd_n))
    q2, s2, z2 = awq.unpack_inputs_1d(packed, n, gs, herd_n)
    assert np.array_equal(q2, q) and np.array_equal(bf16.bits_of(s2), s) and np.array_equal(z2, z)
    for n2, gs2, h2 in ((512, 64, 8), (128, 128, 1), (4096, 128, 2)):
        q = rng.integers(0, 16, n2).astype(np.uint8)
        z = rng.integers(0, 16, n2 // gs2).astype(np.uint8)
        s = rng.integers(0, 65536, n2 // gs2).astype(np.uint16)
        assert np.array_equal(awq.pack_inputs_1d(q, bf16.from_bits(s), z, n2, gs2, h2), oawq.pack_inputs_1d_loop(q, s, z, n2, gs2, h2))
    with pytest.raises(ValueError):
        awq.pack_inputs_1d(q, bf16.from_bits(s), z, 4096, 128, 3)
