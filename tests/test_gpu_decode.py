"""GPU parity of the decode attention kernel and of a whole decode block against the oracle."""
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


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


@pytest.mark.parametrize("n_heads,n_kv,hd,max_seq,positions", [
    (8, 2, 64, 64, [0, 1, 7, 31, 63]),            # one chunk
    (32, 8, 64, 2048, [0, 127, 128, 500, 2047]),  # Llama-3.2-1B heads, up to 16 chunks
    (8, 8, 128, 700, [5, 300, 699]),              # no grouping, head_dim 128, ragged chunks
    (16, 2, 128, 4500, [4499]),                   # group 8, chunk count capped at 32
    (4, 2, 64, 300, [299]),                       # group 2
])
def test_decode_attention(ops, n_heads, n_kv, hd, max_seq, positions):
    rng = np.random.default_rng(n_heads * 1000 + hd)
    lut = odec.generate_rope_lut(hd, 500000.0, max_seq)
    k_cache = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    v_cache = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    dk, dv, dlut = dev(k_cache), dev(v_cache), dev(lut)
    for pos in positions:
        print(f"attention heads={n_heads}/{n_kv} hd={hd} pos={pos}", flush=True)
        qkv = f32_to_bf16_bits(rng.standard_normal((n_heads + 2 * n_kv) * hd).astype(np.float32))
        out = ops.decode_attention(dev(qkv), dlut[pos], dk, dv, pos, n_heads)
        torch.cuda.synchronize()
        nq, nkv = n_heads * hd, n_kv * hd
        q_r = odec.rope_halfsplit(qkv[:nq].reshape(n_heads, hd), lut[pos]).reshape(-1)
        k_r = odec.rope_halfsplit(qkv[nq:nq + nkv].reshape(n_kv, hd), lut[pos])
        k_cache[:, pos, :] = k_r
        v_cache[:, pos, :] = qkv[nq + nkv:].reshape(n_kv, hd)
        # the append is bit-exact (RoPE is two exact products and one add in fp32, one rounding)
        assert np.array_equal(bits(dk)[:, pos, :], k_cache[:, pos, :])
        assert np.array_equal(bits(dv)[:, pos, :], v_cache[:, pos, :])
        assert np.array_equal(bits(dk), k_cache) and np.array_equal(bits(dv), v_cache)   # nothing else touched
        want = bf16_bits_to_f32(odec.decode_attention_cpu(q_r, k_cache, v_cache, pos, n_heads, n_kv, hd)).astype(np.float64)
        # fp32 softmax in a different summation order and exp2 instead of exp: 1 bf16 ulp + 2e-3
        assert_bf16_close(bits(out), want, ulps=1.0, atol=2e-3, what=f"attention pos={pos}")


def _layer(E, H, n_heads, n_kv, hd, seed):
    t = {"wq": make_awq(E, n_heads * hd, seed=seed), "wk": make_awq(E, n_kv * hd, seed=seed + 1),
         "wv": make_awq(E, n_kv * hd, seed=seed + 2), "wo": make_awq(n_heads * hd, E, seed=seed + 3),
         "w_gate": make_awq(E, H, seed=seed + 4), "w_up": make_awq(E, H, seed=seed + 5),
         "w_down": make_awq(H, E, seed=seed + 6)}
    rng = np.random.default_rng(seed + 7)
    norm = lambda: f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    return t, norm(), norm()


def test_decode_block_matches_the_oracle_over_several_tokens(ops):
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=1, emb_dim=512, n_heads=8, head_dim=64, n_kv_heads=2, hidden_dim=1024, vocab_size=32)
    max_seq = 160
    t, attn_norm, ffn_norm = _layer(cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, seed=300)
    # scale the projections down so that activations stay O(1) through the block
    small = lambda w: (w[0], w[1], f32_to_bf16_bits(bf16_bits_to_f32(w[2]) * 0.05))
    t = {k: small(v) for k, v in t.items()}
    host = weights.LayerWeights(attn_norm=attn_norm, ffn_norm=ffn_norm, **t)
    layer = decode.prepare_layer(host)
    l1 = {k: oawq.repack_hf_awq_linear(*v, 128) for k, v in t.items()}
    l1.update(attn_norm=attn_norm, ffn_norm=ffn_norm)
    lut_bits = odec.generate_rope_lut(cfg.head_dim, cfg.rope_base, max_seq)
    lut = decode.generate_rope_lut(cfg, max_seq)
    assert np.array_equal(bits(lut), lut_bits)
    (kc, vc), = decode.new_kv_cache(cfg, max_seq)
    kc_ref = np.zeros((cfg.n_kv_heads, max_seq, cfg.head_dim), np.uint16)
    vc_ref = np.zeros_like(kc_ref)
    rng = np.random.default_rng(9)
    for pos in list(range(6)) + [130]:
        print(f"decode block pos={pos}", flush=True)
        if pos == 130:   # jump ahead: fill the gap identically on both sides
            fill = f32_to_bf16_bits(rng.standard_normal((2, cfg.n_kv_heads, 124, cfg.head_dim)).astype(np.float32))
            kc_ref[:, 6:130], vc_ref[:, 6:130] = fill[0], fill[1]
            kc[:, 6:130] = dev(fill[0])
            vc[:, 6:130] = dev(fill[1])
        x = make_x((cfg.emb_dim,), seed=400 + pos)
        y = decode.run_decode_block(dev(x), layer, cfg, kc, vc, pos, lut)
        torch.cuda.synchronize()
        want = odec.decode_block_reference(x, l1, kc_ref, vc_ref, pos, lut_bits, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim)
        got_f, want_f = bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(want)
        # the reference's own block gate, then a tighter bound: a few bf16 ulps of the output scale
        assert oref.check_outputs(got_f, want_f, rtol=0.2, atol=2.0, min_correlation=0.99)
        assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), np.max(np.abs(got_f - want_f))
        # caches agree up to one-ulp flips that the RMSNorm prologue's rounding may cause in K/V
        kd = np.abs(bf16_bits_to_f32(bits(kc)[:, pos]) - bf16_bits_to_f32(kc_ref[:, pos]))
        assert np.all(kd <= 2 * bf16_ulp(bf16_bits_to_f32(kc_ref[:, pos])) + 2e-2), kd.max()
        # keep both sides in lock step for the following positions
        kc[:, pos] = dev(kc_ref[:, pos])
        vc[:, pos] = dev(vc_ref[:, pos])


def test_decode_token_runs_a_two_layer_model(ops):
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64, n_kv_heads=2, hidden_dim=512, vocab_size=64)
    layers = []
    for i in range(cfg.n_layers):
        t, an, fn = _layer(cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, seed=500 + 10 * i)
        t = {k: (v[0], v[1], f32_to_bf16_bits(bf16_bits_to_f32(v[2]) * 0.05)) for k, v in t.items()}
        layers.append(decode.prepare_layer(weights.LayerWeights(attn_norm=an, ffn_norm=fn, **t)))
    g = torch.Generator(device="cuda").manual_seed(1)
    embed = torch.randn((cfg.vocab_size, cfg.emb_dim), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = torch.ones(cfg.emb_dim, device="cuda", dtype=torch.bfloat16)
    lut = decode.generate_rope_lut(cfg, 32)
    cache = decode.new_kv_cache(cfg, 32)
    tok = 3
    for pos in range(4):
        print(f"decode token pos={pos}", flush=True)
        logits = decode.decode_token(tok, layers, embed, final_norm, embed, cfg, cache, pos, lut)
        assert logits.shape == (cfg.vocab_size,) and torch.isfinite(logits).all()
        tok = int(torch.argmax(logits))
    assert float(cache[1][0][:, :4].float().abs().sum()) > 0 and float(cache[1][0][:, 4:].float().abs().sum()) == 0


def test_decode_greedy_matches_token_by_token_decoding(ops):
    """The device-side greedy loop produces the tokens that decode_token + a host argmax produce."""
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64, n_kv_heads=2, hidden_dim=512, vocab_size=200)
    layers = []
    for i in range(cfg.n_layers):
        t, an, fn = _layer(cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, seed=700 + 10 * i)
        t = {k: (v[0], v[1], f32_to_bf16_bits(bf16_bits_to_f32(v[2]) * 0.05)) for k, v in t.items()}
        layers.append(decode.prepare_layer(weights.LayerWeights(attn_norm=an, ffn_norm=fn, **t)))
    g = torch.Generator(device="cuda").manual_seed(2)
    embed = torch.randn((cfg.vocab_size, cfg.emb_dim), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = (torch.randn(cfg.emb_dim, device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)
    lut = decode.generate_rope_lut(cfg, 32)
    n = 6
    print("greedy loop, token by token", flush=True)
    cache = decode.new_kv_cache(cfg, 32)
    tok, want = 5, []
    for pos in range(n):
        logits, best = decode.decode_token(tok, layers, embed, final_norm, embed, cfg, cache, pos, lut, return_argmax=True)
        tok = int(torch.argmax(logits))
        assert tok == int(best.item())
        want.append(tok)
    print("greedy loop, on the device", flush=True)
    cache2 = decode.new_kv_cache(cfg, 32)
    first = torch.tensor([5], dtype=torch.int32, device="cuda")
    got = decode.decode_greedy(first, n, layers, embed, final_norm, embed, cfg, cache2, 0, lut)
    torch.cuda.synchronize()
    assert got.tolist() == want
    for (k1, v1), (k2, v2) in zip(cache, cache2):
        assert torch.equal(k1, k2) and torch.equal(v1, v2)


def test_prefill_then_decode_agrees_with_token_by_token_decoding(ops):
    """The prompt pass (tiled GEMMs, causal attention) and the decode path (streaming GEMVs, single-query
    attention) are two implementations of the same model: after the same 20 tokens their KV caches and
    last-position logits agree to bf16 noise, and decoding continues from either."""
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64, n_kv_heads=2, hidden_dim=512, vocab_size=300)
    layers = []
    for i in range(cfg.n_layers):
        t, an, fn = _layer(cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, seed=900 + 10 * i)
        t = {k: (v[0], v[1], f32_to_bf16_bits(bf16_bits_to_f32(v[2]) * 0.05)) for k, v in t.items()}
        layers.append(decode.prepare_layer(weights.LayerWeights(attn_norm=an, ffn_norm=fn, **t)))
    g = torch.Generator(device="cuda").manual_seed(3)
    embed = torch.randn((cfg.vocab_size, cfg.emb_dim), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = (torch.randn(cfg.emb_dim, device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)
    lut = decode.generate_rope_lut(cfg, 64)
    prompt = torch.randint(0, cfg.vocab_size, (20,), device="cuda", generator=g, dtype=torch.int64)
    print("prefill of 20 tokens", flush=True)
    cache_p = decode.new_kv_cache(cfg, 64)
    logits_p, best_p = decode.prefill(prompt, layers, embed, final_norm, embed, cfg, cache_p, lut)
    print("the same 20 tokens one by one", flush=True)
    cache_d = decode.new_kv_cache(cfg, 64)
    for pos, tok in enumerate(prompt.tolist()):
        logits_d = decode.decode_token(tok, layers, embed, final_norm, embed, cfg, cache_d, pos, lut)
    torch.cuda.synchronize()
    assert int(best_p.item()) == int(torch.argmax(logits_p))
    scale = float(logits_d.abs().max())
    assert float((logits_p - logits_d).abs().max()) <= 0.05 * scale, float((logits_p - logits_d).abs().max()) / scale
    for (kp, vp), (kd, vd) in zip(cache_p, cache_d):
        for a, b in ((kp, kd), (vp, vd)):
            assert float((a[:, :20].float() - b[:, :20].float()).abs().max()) <= 0.05 * float(b.float().abs().max())
            assert float(a[:, 20:].float().abs().sum()) == 0
    # decoding goes on from the prefilled caches
    nxt = decode.decode_token(int(best_p.item()), layers, embed, final_norm, embed, cfg, cache_p, 20, lut)
    ref = decode.decode_token(int(best_p.item()), layers, embed, final_norm, embed, cfg, cache_d, 20, lut)
    assert float((nxt - ref).abs().max()) <= 0.05 * float(ref.abs().max())


def test_generate_is_prefill_plus_greedy_decoding_and_stops_at_eos(ops):
    """generate() against its parts: the first token is the prompt pass's argmax, the rest equals a token-by-token
    greedy loop from the prefilled caches; the device loop and the streaming loop agree; an end-of-sequence id ends
    the output with that id."""
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=2, emb_dim=256, n_heads=4, head_dim=64, n_kv_heads=2, hidden_dim=512, vocab_size=300)
    layers = []
    for i in range(cfg.n_layers):
        t, an, fn = _layer(cfg.emb_dim, cfg.hidden_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, seed=1100 + 10 * i)
        t = {k: (v[0], v[1], f32_to_bf16_bits(bf16_bits_to_f32(v[2]) * 0.05)) for k, v in t.items()}
        layers.append(decode.prepare_layer(weights.LayerWeights(attn_norm=an, ffn_norm=fn, **t)))
    g = torch.Generator(device="cuda").manual_seed(5)
    embed = torch.randn((cfg.vocab_size, cfg.emb_dim), device="cuda", generator=g).to(torch.bfloat16)
    final_norm = (torch.randn(cfg.emb_dim, device="cuda", generator=g) * 0.1 + 1.0).to(torch.bfloat16)
    lut = decode.generate_rope_lut(cfg, 64)
    prompt = torch.randint(0, cfg.vocab_size, (12,), device="cuda", generator=g, dtype=torch.int64).tolist()
    n = 9
    print("generate: device loop", flush=True)
    got = decode.generate(prompt, layers, embed, final_norm, embed, cfg, lut, n_tokens=n, eos_token_ids=())
    assert len(got) == n + 1
    print("generate: reference loop from its parts", flush=True)
    cache = decode.new_kv_cache(cfg, len(prompt) + n)
    _, first = decode.prefill(torch.tensor(prompt, device="cuda"), layers, embed, final_norm, embed, cfg, cache, lut)
    want = [int(first.item())]
    for i in range(n):
        logits = decode.decode_token(want[-1], layers, embed, final_norm, embed, cfg, cache, len(prompt) + i, lut)
        want.append(int(torch.argmax(logits)))
    assert got == want
    print("generate: streaming", flush=True)
    seen = []
    streamed = decode.generate(prompt, layers, embed, final_norm, embed, cfg, lut, n_tokens=n, eos_token_ids=(), on_token=seen.append)
    assert streamed == want and seen == want
    # an end-of-sequence id ends the output at its first occurrence among the decoded tokens, in both modes (the
    # prompt pass's own token is not tested, as in the reference's loop)
    for eos in (want[1], want[-1]):
        cut = next(i for i in range(1, len(want)) if want[i] == eos)
        for cb in (None, lambda t: None):
            out = decode.generate(prompt, layers, embed, final_norm, embed, cfg, lut, n_tokens=n, eos_token_ids=(eos,), on_token=cb)
            assert out == want[:cut + 1]
    with pytest.raises(ValueError):
        decode.generate(prompt, layers, embed, final_norm, embed, cfg, lut, n_tokens=60)


@pytest.mark.parametrize("n_heads,n_kv,hd,H,max_seq,positions", [
    (32, 8, 128, 14336, 2048, [0, 63, 64, 500, 2047]),   # Llama-3-8B layer: fused from position 64 on (2 .. 32 chunks)
    (32, 8, 64, 8192, 2048, [100, 2047]),                # Llama-3.2-1B layer
    (8, 2, 64, 1024, 300, [10, 299]),                    # small E
])
def test_attention_and_block_in_one_call_equal_the_two_calls(ops, n_heads, n_kv, hd, H, max_seq, positions):
    """w4a16_decode_attn_o_gemv_ffn_bf16 against w4a16_decode_attention_bf16 + w4a16_o_gemv_ffn_bf16: the same output bit
    for bit (the O projection's merge of the attention partials repeats the merge kernel's arithmetic in its order), the
    same cache update, with the merge launch kept (tune attn_fuse = 0) and dropped."""
    E = n_heads * hd
    rng = np.random.default_rng(n_heads + hd + H)
    wo, wg, wu, wd = (tuple(map(dev, make_awq(a, b, seed=50 + i))) for i, (a, b) in enumerate([(E, E), (E, H), (E, H), (H, E)]))
    small = lambda w: (w[0], w[1], (w[2].float() * 0.05).to(torch.bfloat16))
    wo, wg, wu, wd = map(small, (wo, wg, wu, wd))
    norm_w = dev(f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32)))
    lut = dev(odec.generate_rope_lut(hd, 500000.0, max_seq))
    kc0 = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    vc0 = f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32))
    for pos in positions:
        print(f"attention + block in one call: heads {n_heads}/{n_kv} hd={hd} pos={pos}", flush=True)
        qkv = dev(make_x(((n_heads + 2 * n_kv) * hd,), seed=pos + 1))
        x_res = dev(make_x((E,), seed=pos + 2))
        ka, va = dev(kc0), dev(vc0)
        attn = ops.decode_attention(qkv, lut[pos], ka, va, pos, n_heads)
        want = ops.o_gemv_ffn(attn, x_res, norm_w, wo, wg, wu, wd)
        for fuse in (1, 0):
            ops.tune("attn_fuse", fuse)
            kb, vb = dev(kc0), dev(vc0)
            got = ops.decode_attn_o_gemv_ffn(qkv, lut[pos], kb, vb, pos, n_heads, x_res, norm_w, wo, wg, wu, wd)
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (pos, fuse)
            assert torch.equal(kb.view(torch.int16), ka.view(torch.int16)) and torch.equal(vb.view(torch.int16), va.view(torch.int16))
        ops.tune("attn_fuse", 1)


@pytest.mark.parametrize("n_heads,n_kv,hd,H", [(32, 8, 128, 14336), (32, 8, 64, 8192), (8, 2, 64, 1024)])
def test_sum_of_squares_chained_into_the_next_norm(ops, n_heads, n_kv, hd, H):
    """The block's y_sumsq is the sum of squares of its bf16 output per 256-column tile, and w4a16_rms_gemv fed with it
    equals the plain call up to the summation order of the mean (one-ulp flips of the normalised vector)."""
    E, pos, max_seq = n_heads * hd, 70, 128
    rng = np.random.default_rng(E + H)
    small = lambda w: (w[0], w[1], (w[2].float() * 0.05).to(torch.bfloat16))
    wo, wg, wu, wd = (small(tuple(map(dev, make_awq(a, b, seed=80 + i)))) for i, (a, b) in enumerate([(E, E), (E, H), (E, H), (H, E)]))
    wq = tuple(map(dev, make_awq(E, 512, seed=90)))
    norm_w = dev(f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32)))
    lut = dev(odec.generate_rope_lut(hd, 500000.0, max_seq))
    kc = dev(f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32)))
    vc = dev(f32_to_bf16_bits(rng.standard_normal((n_kv, max_seq, hd)).astype(np.float32)))
    qkv, x_res = dev(make_x(((n_heads + 2 * n_kv) * hd,), seed=3)), dev(make_x((E,), seed=4))
    print(f"chained sum of squares E={E} H={H}", flush=True)
    y, sumsq = ops.decode_attn_o_gemv_ffn(qkv, lut[pos], kc.clone(), vc.clone(), pos, n_heads, x_res, norm_w, wo, wg, wu, wd,
                                          return_sumsq=True)
    torch.cuda.synchronize()
    want = (y.float().double() ** 2).reshape(E // 256, 256).sum(dim=1)
    assert sumsq.shape == (E // 256,) and torch.allclose(sumsq.double(), want, rtol=1e-5, atol=0)
    # 128-column tiles (tuning key) must not change the chain: launches that leave or take sums of squares keep
    # their 256-column tiles, one float per tile in a buffer of E / 256
    ops.tune("gemv_lw", 1)
    try:
        y_lw, sumsq_lw = ops.decode_attn_o_gemv_ffn(qkv, lut[pos], kc.clone(), vc.clone(), pos, n_heads, x_res, norm_w, wo, wg, wu, wd,
                                                    return_sumsq=True)
        chained_lw = ops.w4a16_rms_gemv(y_lw, norm_w, *wq, x_sumsq=sumsq_lw)
        torch.cuda.synchronize()
    finally:
        ops.tune("gemv_lw", 0)
    assert torch.equal(y_lw.view(torch.int16), y.view(torch.int16)) and torch.equal(sumsq_lw, sumsq)
    plain = ops.w4a16_rms_gemv(y, norm_w, *wq)
    chained = ops.w4a16_rms_gemv(y, norm_w, *wq, x_sumsq=sumsq)
    torch.cuda.synchronize()
    assert torch.equal(chained_lw.view(torch.int16), chained.view(torch.int16))
    p64, c64 = plain.float().double().cpu().numpy(), chained.float().double().cpu().numpy()
    assert np.max(np.abs(p64 - c64)) <= 2 * 2.0**-8 * np.max(np.abs(p64))
    assert np.mean(p64 != c64) < 0.2
