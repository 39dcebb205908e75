"""GPU parity of the KernelCache boundary: the reference's decode loop driven through load_and_run
with the reference's packed decode buffers, against the oracle chain."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close, bf16_ulp, make_awq, make_x
from oracle import awq as oawq, decode as odec, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("rows,dim", [(32, 64), (8, 64), (5, 128), (1, 16), (300, 256)])
def test_rope_halfsplit_is_bit_exact(rows, dim):
    from air_hip import ops

    rng = np.random.default_rng(rows * 1000 + dim)
    x = f32_to_bf16_bits(rng.standard_normal((rows, dim)).astype(np.float32))
    ang = rng.uniform(-np.pi, np.pi, size=(rows, dim // 2))
    lut = f32_to_bf16_bits(np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32))
    print(f"rope rows={rows} dim={dim}", flush=True)
    got = bits(ops.rope_halfsplit(dev(x), dev(lut)))
    assert np.array_equal(got, odec.rope_rows(x, lut))
    # a rotation by zero returns x, by a quarter turn swaps the halves with a sign
    ident = f32_to_bf16_bits(np.concatenate([np.ones((rows, dim // 2)), np.zeros((rows, dim // 2))], axis=1).astype(np.float32))
    assert np.array_equal(bits(ops.rope_halfsplit(dev(x), dev(ident))), x)
    quarter = f32_to_bf16_bits(np.concatenate([np.zeros((rows, dim // 2)), np.ones((rows, dim // 2))], axis=1).astype(np.float32))
    q = bf16_bits_to_f32(bits(ops.rope_halfsplit(dev(x), dev(quarter))))
    xf = bf16_bits_to_f32(x)
    assert np.array_equal(q[:, :dim // 2], -xf[:, dim // 2:]) and np.array_equal(q[:, dim // 2:], xf[:, :dim // 2])


def _model(E, H, nh, nkv, hd, seed):
    from air_hip import weights

    t = {"wq": make_awq(E, nh * hd, seed=seed), "wk": make_awq(E, nkv * hd, seed=seed + 1),
         "wv": make_awq(E, nkv * hd, seed=seed + 2), "wo": make_awq(nh * hd, E, seed=seed + 3),
         "w_gate": make_awq(E, H, seed=seed + 4), "w_up": make_awq(E, H, seed=seed + 5),
         "w_down": make_awq(H, E, seed=seed + 6)}
    small = lambda w: (w[0], w[1], f32_to_bf16_bits(bf16_bits_to_f32(w[2]) * 0.05))
    t = {k: small(v) for k, v in t.items()}
    rng = np.random.default_rng(seed + 7)
    norm = lambda: f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    attn_norm, ffn_norm = norm(), norm()
    host = weights.LayerWeights(attn_norm=attn_norm, ffn_norm=ffn_norm, **t)
    l1 = {k: oawq.repack_hf_awq_linear(*v, 128) for k, v in t.items()}
    l1.update(attn_norm=attn_norm, ffn_norm=ffn_norm)
    return host, l1


def _decode_block_through_cache(cache, x, packed, attn_norm, ffn_norm, cfg, k_cache, v_cache, pos, lut_bits, layer_idx):
    """The call sequence of run_decode_block (llama32_1b_int4_decode.py:176-313): two load_and_run calls with
    the KV-cache update and the host attention between them."""
    from air_hip import bf16

    E, H, nh, nkv, hd = cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
    kv = nkv * hd
    z = lambda n: bf16.from_bits(np.zeros(n, np.uint16))
    lut_row = lut_bits[pos:pos + 1]
    r = cache.load_and_run(
        "rms_qkv_int4_rope", {}, bf16.from_bits(x), bf16.from_bits(attn_norm), z(E), packed["_wq_packed"], z(E),
        packed["_wk_packed"], z(kv), packed["_wv_packed"], z(kv), bf16.from_bits(np.tile(lut_row, (nh, 1)).reshape(-1)),
        bf16.from_bits(np.tile(lut_row, (nkv, 1)).reshape(-1)), z(E), z(kv),
        output_indices=[8, 11, 12], static_input_indices={1, 3, 5, 7}, intermediate_indices={2, 4, 6, 8, 11, 12},
        bo_key=f"rms_qkv_int4_rope_L{layer_idx}")
    assert [a.size for a in r] == [0] * 8 + [kv, 0, 0, E, kv]
    v, q_roped, k_roped = (np.asarray(r[i]).view(np.uint16) for i in (8, 11, 12))
    k_cache[:, pos, :] = k_roped.reshape(nkv, hd)
    v_cache[:, pos, :] = v.reshape(nkv, hd)
    attn_out = odec.decode_attention_cpu(q_roped, k_cache, v_cache, pos, nh, nkv, hd)
    rms_buf = bf16.from_bits(np.stack([np.zeros(E, np.uint16), ffn_norm]))
    r = cache.load_and_run(
        "o_gemv_ffn_int4", {}, packed["_wo_packed"], bf16.from_bits(attn_out), z(E), bf16.from_bits(x), z(E), z(E),
        rms_buf, packed["_wgateup_packed"], z(H), z(16), z(H), z(H), packed["_wdown_packed"], z(E), z(E),
        output_indices=[14], static_input_indices={0, 6, 7, 12}, intermediate_indices={2, 4, 5, 8, 9, 10, 11, 13, 14},
        bo_key=f"o_gemv_ffn_int4_L{layer_idx}")
    assert isinstance(r[14], bf16.BF16Array) and r[14].shape == (E,) and r[13].size == 0
    return np.asarray(r[14]).view(np.uint16), (q_roped, k_roped, v)


@pytest.mark.parametrize("stream_order", [True, False])
def test_decode_blocks_through_the_kernel_cache_match_the_oracle(stream_order):
    """stream_order: the static weight slots are kept in stream order and the whole-K launches run (the default);
    False keeps AutoAWQ triples for the checkpoint-layout kernels."""
    from air_hip import cache as kc, ops, weights

    cfg = weights.LlamaConfig(n_layers=2, emb_dim=512, n_heads=8, head_dim=64, n_kv_heads=2, hidden_dim=1024, vocab_size=32)
    E, H, nh, nkv, hd = cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
    max_seq = 16
    models = [_model(E, H, nh, nkv, hd, seed=500 + 20 * i) for i in range(cfg.n_layers)]
    packed = [weights.reference_decode_buffers(host, k_chunk=E) for host, _ in models]
    cache = kc.KernelCache(profiler=kc.Profiler(enabled=True), stream_order=stream_order)
    cache.compile_and_cache("rms_qkv_int4_rope", kc.build_rms_qkv_int4_rope_module(E, nkv * hd, nh, nkv, hd, k_chunk=E), {})
    cache.compile_and_cache("o_gemv_ffn_int4", kc.build_o_gemv_ffn_int4_module(E, H, k_chunk=E), {})
    lut_bits = odec.generate_rope_lut(hd, cfg.rope_base, max_seq)
    caches = [(np.zeros((nkv, max_seq, hd), np.uint16), np.zeros((nkv, max_seq, hd), np.uint16)) for _ in models]
    ref_caches = [(k.copy(), v.copy()) for k, v in caches]
    for pos in range(4):
        x = make_x((E,), seed=700 + pos)
        x_ref = x.copy()
        for li, ((host, l1), pk) in enumerate(zip(models, packed)):
            print(f"kernel cache decode pos={pos} layer={li}", flush=True)
            want_qkv = odec.rms_qkv_rope_reference(x_ref, l1["attn_norm"], l1["wq"], l1["wk"], l1["wv"], lut_bits[pos], nh, nkv, hd)
            y, got_qkv = _decode_block_through_cache(cache, x_ref, pk, host.attn_norm, host.ffn_norm, cfg, *caches[li], pos, lut_bits, li)
            for got, want in zip(got_qkv, want_qkv):
                d = np.abs(bf16_bits_to_f32(got) - bf16_bits_to_f32(want))
                assert np.all(d <= 2 * bf16_ulp(bf16_bits_to_f32(want)) + 2e-2), d.max()
            want = odec.decode_block_reference(x_ref, l1, *ref_caches[li], pos, lut_bits, nh, nkv, hd)
            got_f, want_f = bf16_bits_to_f32(y), bf16_bits_to_f32(want)
            assert oref.check_outputs(got_f, want_f, rtol=0.2, atol=2.0, min_correlation=0.99)
            assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), np.max(np.abs(got_f - want_f))
            # both sides continue from the oracle's state so that one-ulp differences do not compound
            caches[li][0][:, pos], caches[li][1][:, pos] = ref_caches[li][0][:, pos], ref_caches[li][1][:, pos]
            x_ref = want
    assert len(cache.profiler.kernel_times["o_gemv_ffn_int4"]) == 8
    kept = [cache._cached_bos["rms_qkv_int4_rope_L1"]["wqkv"], cache._cached_bos["o_gemv_ffn_int4_L0"]["wdown"],
            *cache._cached_bos["o_gemv_ffn_int4_L1"]["wgateup"]]
    assert all(isinstance(w, ops.StreamWeight) == stream_order for w in kept)
    bd = cache.profiler.kernel_breakdowns["o_gemv_ffn_int4"]
    # static slots are written on the first call of a bo_key only: 3 packed buffers + the RMS buffer, then 2 vectors
    assert bd[0]["n_written"] == 6 and bd[1]["n_written"] == 6 and bd[2]["n_written"] == 2 and bd[-1]["n_written"] == 2


def test_static_slots_are_written_once_per_bo_key_and_other_outputs_can_be_read_back():
    from air_hip import bf16, cache as kc, weights

    E, H = 256, 512
    host_a, l1_a = _model(E, H, 4, 2, 64, seed=900)
    host_b, l1_b = _model(E, H, 4, 2, 64, seed=950)
    pk_a = weights.reference_decode_buffers(host_a, k_chunk=E)
    pk_b = weights.reference_decode_buffers(host_b, k_chunk=E)
    cache = kc.KernelCache()
    cache.compile_and_cache("o_gemv_ffn_int4", kc.build_o_gemv_ffn_int4_module(E, H, k_chunk=E), {})
    attn, xres = make_x((E,), seed=1), make_x((E,), seed=2)
    z = lambda n: bf16.from_bits(np.zeros(n, np.uint16))

    def call(pk, host, key):
        rms_buf = bf16.from_bits(np.stack([np.zeros(E, np.uint16), host.ffn_norm]))
        r = cache.load_and_run("o_gemv_ffn_int4", {}, pk["_wo_packed"], bf16.from_bits(attn), z(E), bf16.from_bits(xres),
                               z(E), z(E), rms_buf, pk["_wgateup_packed"], z(H), z(16), z(H), z(H), pk["_wdown_packed"],
                               z(E), z(E), output_indices=[6, 11, 14], static_input_indices={0, 6, 7, 12},
                               intermediate_indices={11, 14}, bo_key=key)
        return [np.asarray(r[i]).view(np.uint16) for i in (6, 11, 14)]

    rms_a, h_a, y_a = call(pk_a, host_a, "L0")
    res1, h, y = oref.o_gemv_ffn_staged_reference(l1_a["wo"], l1_a["w_gate"], l1_a["w_up"], l1_a["w_down"], attn, xres,
                                                  host_a.ffn_norm)
    assert np.array_equal(rms_a[E:], host_a.ffn_norm)
    for got, want in ((rms_a[:E], res1), (h_a, h), (y_a, y)):
        d = np.abs(bf16_bits_to_f32(got) - bf16_bits_to_f32(want))
        assert np.all(d <= 8 * 2.0**-8 * np.max(np.abs(bf16_bits_to_f32(want)))), d.max()
    # the same bo_key keeps layer A's weights whatever is passed in the static slots afterwards ...
    _, _, y_again = call(pk_b, host_b, "L0")
    assert np.array_equal(y_again, y_a)
    # ... and another bo_key gets its own
    _, _, y_b = call(pk_b, host_b, "L1")
    assert not np.array_equal(y_b, y_a)
    with pytest.raises(Exception, match="not outputs"):
        cache.load_and_run("o_gemv_ffn_int4", {}, pk_a["_wo_packed"], bf16.from_bits(attn), z(E), bf16.from_bits(xres), z(E),
                           z(E), bf16.from_bits(np.zeros((2, E), np.uint16)), pk_a["_wgateup_packed"], z(H), z(16), z(H),
                           z(H), pk_a["_wdown_packed"], z(E), z(E), output_indices=[2], bo_key="L2")


def test_lm_head_partitions_through_the_kernel_cache():
    from air_hip import bf16, cache as kc

    E, n_part, parts, vocab = 256, 512, 3, 1300
    rng = np.random.default_rng(5)
    w = f32_to_bf16_bits((rng.standard_normal((vocab, E)) * 0.05).astype(np.float32))
    x = make_x((E,), seed=3)
    cache = kc.KernelCache()
    cache.compile_and_cache("lm_head_gemv", kc.build_lm_head_gemv_module(E, parts, n_part), {})
    args = [bf16.from_bits(x)]
    for p in range(parts):   # zero-padded row blocks, as _preload_decode_weights builds them
        blk = np.zeros((n_part, E), np.uint16)
        rows = w[p * n_part:min((p + 1) * n_part, vocab)]
        blk[:rows.shape[0]] = rows
        args += [bf16.from_bits(blk), bf16.from_bits(np.zeros(n_part, np.uint16))]
    r = cache.load_and_run("lm_head_gemv", {}, *args, output_indices=[2 + 2 * p for p in range(parts)],
                           static_input_indices={1 + 2 * p for p in range(parts)},
                           intermediate_indices={2 + 2 * p for p in range(parts)})
    logits = np.concatenate([np.asarray(r[2 + 2 * p]).view(np.uint16) for p in range(parts)])[:vocab]
    want = bf16_bits_to_f32(w).astype(np.float64) @ bf16_bits_to_f32(x).astype(np.float64)
    assert_bf16_close(logits, want, ulps=1.0, atol=2e-3, what="lm_head partitions")
    assert int(np.argmax(bf16_bits_to_f32(logits))) == odec.lm_head_reference(x, None, w)[1]


@pytest.mark.parametrize("stream_order,M,E,H,nh,nkv", [(True, 72, 256, 512, 4, 2), (False, 72, 256, 512, 4, 2), (True, 40, 384, 640, 6, 3)])
def test_prompt_layer_through_the_kernel_cache_matches_the_oracle(stream_order, M, E, H, nh, nkv):
    """The call sequence of _run_layer_int4 (llama32_1b_int4_prefill.py:241-364): rms_gemms_rope_int4, flash_attn,
    o_ffn_int4, with the packed GEMM buffers awq_pack_for_npu makes, stage by stage against the oracle; on the
    stream-order copies of the weights (the default) and on the AutoAWQ triples; an embedding width that is not a
    whole number of group pairs (384) keeps the triples whatever the setting."""
    from air_hip import bf16, cache as kc, ops, weights

    hd = 64
    kv = nkv * hd
    host, l1 = _model(E, H, nh, nkv, hd, seed=1200)
    # larger Q/K/V scales than the decode tests use: attention scores with some spread
    big = lambda w: (w[0], w[1], f32_to_bf16_bits(bf16_bits_to_f32(w[2]) * 5.0))
    for f in ("wq", "wk", "wv"):
        setattr(host, f, big(getattr(host, f)))
        l1[f] = oawq.repack_hf_awq_linear(*getattr(host, f), 128)
    packed = weights.reference_prefill_buffers(host, n_tile=16, k_chunk=128)
    cache = kc.KernelCache(stream_order=stream_order)
    cache.compile_and_cache("rms_gemms_rope_int4", kc.build_rms_gemms_rope_int4_module(M, E, kv, nh, nkv, hd, tile_n=16), {})
    cache.compile_and_cache("flash_attn", kc.build_attn(lk=M, lkp=hd, lq=M, lqp=256, dk=hd, dv=hd, num_heads=nh,
                                                        num_kv_heads=nkv, causal=True), {})
    cache.compile_and_cache("o_ffn_int4", kc.build_o_ffn_int4_module(M, E, H, tile_n=16), {})
    lut = odec.generate_rope_lut(hd, 500000.0, M)
    x = make_x((M, E), seed=1300)
    z = lambda *shape: bf16.from_bits(np.zeros(shape, np.uint16))
    f = lambda b: bf16_bits_to_f32(np.asarray(b).view(np.uint16)).astype(np.float64)
    print("kernel cache prompt layer: rms_gemms_rope_int4", flush=True)
    r = cache.load_and_run(
        "rms_gemms_rope_int4", {}, bf16.from_bits(x), bf16.from_bits(host.attn_norm), z(M, E), packed["wq"], z(M, E),
        packed["wk"], z(M, kv), packed["wv"], z(M, kv), bf16.from_bits(np.repeat(lut, nh, axis=0).reshape(-1)),
        bf16.from_bits(np.repeat(lut, nkv, axis=0).reshape(-1)), z(M, E), z(M, kv),
        output_indices=[2, 4, 6, 8, 11, 12], static_input_indices={1, 3, 5, 7, 9, 10},
        intermediate_indices={2, 4, 6, 8, 11, 12}, bo_key="rms_int4_L0")
    v, q_roped, k_roped = (np.asarray(r[i]).view(np.uint16) for i in (8, 11, 12))
    want = odec.prefill_rms_qkv_rope_reference(x, host.attn_norm, l1["wq"], l1["wk"], l1["wv"], lut, 0, nh, nkv, hd)
    got = np.concatenate([q_roped.reshape(M, E), k_roped.reshape(M, kv), v.reshape(M, kv)], axis=1)
    assert np.max(np.abs(f(got) - f(want))) <= 4 * 2.0**-8 * np.max(np.abs(f(want)))
    # the diagnostic slots: normed input, and Q before the rotation (at this M the plain product comes from the
    # streaming kernel, whose weights are not rounded to bf16 first: rotating it gives slot 11 up to one-ulp flips)
    assert np.mean(np.asarray(r[2]).view(np.uint16).reshape(M, E) != oref.rms_norm_rows_bf16(x, host.attn_norm, 1e-5)) < 0.02
    q_plain = np.asarray(r[4]).view(np.uint16).reshape(M * nh, hd)
    rerot = odec.rope_rows(q_plain, np.repeat(lut, nh, axis=0)).reshape(-1)
    assert np.max(np.abs(f(rerot) - f(q_roped))) <= 2 * 2.0**-8 * np.max(np.abs(f(q_roped)))

    print("kernel cache prompt layer: flash_attn", flush=True)
    r = cache.load_and_run("flash_attn", {}, bf16.from_bits(q_roped.reshape(M, E)), bf16.from_bits(k_roped.reshape(M, kv)),
                           bf16.from_bits(v.reshape(M, kv)), z(M, E), output_indices=[3], bo_key="flash_attn_L0")
    attn = np.asarray(r[3]).view(np.uint16).reshape(M, E)
    want_attn = odec.prefill_attention_reference(q_roped.reshape(M, E), k_roped.reshape(M, kv), v.reshape(M, kv), nh, nkv)
    tol = bf16_ulp(want_attn) + 2.0**-8 * np.max(np.abs(f(v))) + 1e-3
    assert np.all(np.abs(f(attn) - want_attn) <= tol)

    print("kernel cache prompt layer: o_ffn_int4", flush=True)
    r = cache.load_and_run(
        "o_ffn_int4", {}, bf16.from_bits(attn), packed["wo"], z(M, E), bf16.from_bits(x), z(M, E),
        bf16.from_bits(host.ffn_norm), z(M, E), packed["w_gate"], z(M, H), packed["w_up"], z(M, H), z(M, H),
        packed["w_down"], z(M, E), z(M * E), output_indices=[14], static_input_indices={1, 5, 7, 9, 12},
        intermediate_indices={2, 4, 6, 8, 10, 11, 13, 14}, bo_key="offn_int4_L0")
    assert r[14].shape == (M * E,) and r[4].size == 0
    y = np.asarray(r[14]).view(np.uint16).reshape(M, E)
    want_y, _, _ = oref.o_ffn_int4_prefill_reference(l1["wo"], l1["w_gate"], l1["w_up"], l1["w_down"], attn, x, host.ffn_norm)
    assert oref.check_outputs(f(y), f(want_y), rtol=0.2, atol=2.0, min_correlation=0.99)
    assert np.max(np.abs(f(y) - f(want_y))) <= 8 * 2.0**-8 * np.max(np.abs(f(want_y)))
    kept = [cache._cached_bos["rms_int4_L0"]["wqkv"]] + [cache._cached_bos["offn_int4_L0"][k] for k in ("wo", "wgate", "wup", "wdown")]
    assert all(isinstance(w, ops.StreamWeight) == (stream_order and E % 256 == 0) for w in kept)
