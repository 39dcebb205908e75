"""GPU parity for the Q4NX / Q4_0 block codec: dequant and repack bit-exact against the oracle,
the GEMV within 1 bf16 ulp + 2e-3 of the float64 restatement of the reference kernel's sum
(c += (q.b) * scale + min * sum(b) per 32-column group) and inside the reference's own gate
(rtol 0.1, atol 0.05, r >= 0.999)."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close
from oracle import awq as oawq, q4nx as oq, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


def make(M, K, seed, wild=False):
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, (M, K), dtype=np.uint8)
    if wild:   # any finite bf16 pattern of moderate exponent, both signs
        s = (rng.integers(0x3000, 0x4200, (M, K // 32)) | (rng.integers(0, 2, (M, K // 32)) << 15)).astype(np.uint16)
        m = (rng.integers(0x3000, 0x4200, (M, K // 32)) | (rng.integers(0, 2, (M, K // 32)) << 15)).astype(np.uint16)
    else:      # what a min/max quantiser of N(0, 0.02) weights produces
        s = f32_to_bf16_bits((np.abs(rng.standard_normal((M, K // 32))) * 0.003 + 1e-3).astype(np.float32))
        m = f32_to_bf16_bits((-np.abs(rng.standard_normal((M, K // 32))) * 0.02 - 0.01).astype(np.float32))
    return q, s, m


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
@pytest.mark.parametrize("M,K,wild", [(32, 256, True), (96, 768, False), (512, 2048, True)])
def test_dequant_bit_exact(ops, mode, M, K, wild):
    print(f"q4nx dequant mode={mode} M={M} K={K} wild={wild}", flush=True)
    q, s, m = make(M, K, M + K + mode, wild)
    blocks = oq.pack_matrix(q, s, m)
    out = ops.q4nx_dequant(dev(blocks), M, K, mode)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oq.dequant(blocks, M, K, mode))


def test_dequant_bit_exact_llama8b_projection(ops):
    print("q4nx dequant 4096x4096", flush=True)
    M = K = 4096
    q, s, m = make(M, K, 1)
    blocks = oq.pack_matrix(q, s, m)
    out = ops.q4nx_dequant(dev(blocks), M, K, oq.ADDITIVE)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oq.dequant(blocks, M, K, oq.ADDITIVE))


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
def test_repack_operands(ops, mode):
    print(f"q4nx repack mode={mode}", flush=True)
    M, K = 160, 768
    q, s, m = make(M, K, 20 + mode, wild=True)
    blocks = oq.pack_matrix(q, s, m)
    qw, sc, mn = ops.q4nx_repack(dev(blocks), M, K, mode)
    torch.cuda.synchronize()
    # qweight[k, j] holds rows 8 j .. 8 j + 7 of column k, unsigned, in the AutoAWQ nibble order
    q_u = q ^ 8 if mode == oq.Q4_0 else q
    assert np.array_equal(oawq.unpack_awq_int32(qw.cpu().numpy()), q_u.T)
    assert np.array_equal(bits(sc), s.T)
    sf, mf = bf16_bits_to_f32(s), bf16_bits_to_f32(m)
    want_m = {oq.ADDITIVE: m, oq.SUBTRACTIVE: f32_to_bf16_bits(-(sf * mf)), oq.Q4_0: f32_to_bf16_bits(-8.0 * sf)}[mode]
    assert np.array_equal(bits(mn), want_m.T)


def _gemm_case(ops, rows, M, K, seed, mode=oq.ADDITIVE, residual=False):
    print(f"q4nx gemm rows={rows} M={M} K={K} mode={mode} residual={residual}", flush=True)
    q, s, m = make(M, K, seed)
    rng = np.random.default_rng(seed + 1)
    x = f32_to_bf16_bits(rng.standard_normal((rows, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    qw, sc, mn = ops.q4nx_repack(blocks, M, K, mode)
    res = f32_to_bf16_bits(rng.standard_normal((rows, M)).astype(np.float32)) if residual else None
    y = ops.q4nx_gemm(dev(x), qw, sc, mn, residual=dev(res) if residual else None)
    torch.cuda.synchronize()
    if mode == oq.SUBTRACTIVE:   # the kernel works on the repacked constant term bf16(-s m)
        want = oq.gemv_reference(q, s, bits(mn).T.copy(), x, oq.ADDITIVE)
    else:
        want = oq.gemv_reference(q, s, m, x, mode)
    if residual:
        want = want + bf16_bits_to_f32(res).astype(np.float64)
    got = bits(y)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"q4nx gemm rows={rows} M={M} K={K}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, min_correlation=0.999)
    return got, want


@pytest.mark.parametrize("rows", [1, 3, 4, 7, 16, 17, 40])
def test_gemm_rows(ops, rows):
    _gemm_case(ops, rows, 512, 1024, seed=rows)


@pytest.mark.parametrize("M,K", [(32, 256), (2048, 2048), (1024, 4096), (4096, 14336), (3104, 1280)])
def test_gemv_shapes(ops, M, K):
    _gemm_case(ops, 1, M, K, seed=M + K)


@pytest.mark.parametrize("mode", [oq.SUBTRACTIVE, oq.Q4_0])
def test_gemv_other_conventions(ops, mode):
    _gemm_case(ops, 1, 2048, 2048, seed=30 + mode, mode=mode)


def test_gemv_with_residual(ops):
    _gemm_case(ops, 1, 4096, 4096, seed=40, residual=True)
    _gemm_case(ops, 5, 1024, 512, seed=41, residual=True)


def test_gemv_llama8b_gate_shape_properties(ops):
    """N = 14336 outputs from K = 4096 inputs (the Q4NX Llama-3.1-8B gate projection): against the
    oracle, then determinism, linearity in x (exact for a power-of-two factor) and column independence."""
    M, K = 14336, 4096
    got, want = _gemm_case(ops, 1, M, K, seed=50)
    q, s, m = make(M, K, 50)
    rng = np.random.default_rng(51)
    x = f32_to_bf16_bits(rng.standard_normal((1, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    qw, sc, mn = ops.q4nx_repack(blocks, M, K, oq.ADDITIVE)
    y1 = bits(ops.q4nx_gemm(dev(x), qw, sc, mn))
    x2 = f32_to_bf16_bits(bf16_bits_to_f32(x) * 2.0)
    y2 = bits(ops.q4nx_gemm(dev(x2), qw, sc, mn))
    torch.cuda.synchronize()
    assert np.array_equal(y1, got)                                                    # deterministic
    assert np.array_equal(bf16_bits_to_f32(y2), bf16_bits_to_f32(y1) * 2.0)
    # the first 2048 output features alone (a different K-split, so a different summation order)
    qw_h, sc_h, mn_h = ops.q4nx_repack(blocks[:(2048 // 32) * (K // 256)].contiguous(), 2048, K, oq.ADDITIVE)
    yh = bits(ops.q4nx_gemm(dev(x), qw_h, sc_h, mn_h))
    torch.cuda.synchronize()
    assert_bf16_close(yh, want[:, :2048], ulps=1.0, atol=2e-3, what="first 2048 features alone")
    assert np.mean(yh == y1[:, :2048]) > 0.98


def test_gemv_equals_dequant_then_dense(ops):
    """Same weights through q4nx_dequant + a float64 product: the two GPU paths agree to bf16 rounding
    of the weights (reference gate), tying the repack to the dequant."""
    M, K = 1024, 2048
    q, s, m = make(M, K, 60)
    rng = np.random.default_rng(61)
    x = f32_to_bf16_bits(rng.standard_normal((1, K)).astype(np.float32))
    blocks = dev(oq.pack_matrix(q, s, m))
    W = bf16_bits_to_f32(bits(ops.q4nx_dequant(blocks, M, K, oq.ADDITIVE))).astype(np.float64)
    y = bits(ops.q4nx_gemm(dev(x), *ops.q4nx_repack(blocks, M, K, oq.ADDITIVE)))
    torch.cuda.synchronize()
    want = bf16_bits_to_f32(x).astype(np.float64) @ W.T
    assert oref.check_outputs(bf16_bits_to_f32(y), want.astype(np.float32), rtol=0.1, atol=0.05, min_correlation=0.999)


def test_argument_errors(ops):
    from air_hip import _lib
    blocks = torch.zeros((1, 5120), dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        ops.q4nx_dequant(blocks, 64, 256)
    with pytest.raises(_lib.W4A16Error):
        ops.q4nx_dequant(blocks, 32, 256, mode=3)
    lib = _lib.load_library()
    assert lib.q4nx_repack(None, None, None, None, 32, 256, 0, None) == _lib.ERR_NULL
    assert lib.q4nx_dequant_bf16(blocks.data_ptr(), blocks.data_ptr(), 48, 256, 0, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_gemm_stream_bf16(blocks.data_ptr(), blocks.data_ptr(), None, blocks.data_ptr(), 1, 128, 24, None) == _lib.ERR_SHAPE


# ---- decode-layer entry points on the affine codec ----

def _norm_w(K, seed):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal(K) * 0.1 + 1.0).astype(np.float32))


def _vec(K, seed):
    return f32_to_bf16_bits(np.random.default_rng(seed).standard_normal(K).astype(np.float32))


def _weights(ops, M, K, seed):
    """(host (q, s, m), device (qweight, scales, mins)) of one W[M, K]."""
    w = make(M, K, seed)
    return w, ops.q4nx_repack(dev(oq.pack_matrix(*w)), M, K, oq.ADDITIVE)


@pytest.mark.parametrize("M,K", [(32, 256), (1056, 512), (6144, 4096), (2048, 8192)])
def test_rms_gemv(ops, M, K):
    print(f"q4nx rms_gemv M={M} K={K}", flush=True)
    w, wd = _weights(ops, M, K, seed=M + K)
    x, nw = _vec(K, 70), _norm_w(K, 71)
    y = ops.q4nx_rms_gemv(dev(x), dev(nw), *wd)
    torch.cuda.synchronize()
    # the kernel's normalised vector can differ from the oracle's by one bf16 ulp in single elements
    want = oq.rms_gemv_reference(w, x, nw)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(want), rtol=0.1, atol=0.05, min_correlation=0.999)
    normed = f32_to_bf16_bits(oref.rms_norm_bf16(x, nw))
    y2 = ops.q4nx_gemm(dev(normed), *wd)     # same GEMV without the prologue, fed the oracle's vector
    torch.cuda.synchronize()
    a, b = bf16_bits_to_f32(bits(y)).astype(np.float64), bf16_bits_to_f32(bits(y2)).astype(np.float64)
    from helpers import bf16_ulp
    assert np.all(np.abs(a - b) <= 2 * bf16_ulp(b) + 2e-2), np.abs(a - b).max()


@pytest.mark.parametrize("E,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_o_gemv_ffn_block(ops, E, H):
    print(f"q4nx o_gemv_ffn E={E} H={H}", flush=True)
    wo, wo_d = _weights(ops, E, E, seed=E)
    wg, wg_d = _weights(ops, H, E, seed=E + 1)
    wu, wu_d = _weights(ops, H, E, seed=E + 2)
    wd, wd_d = _weights(ops, E, H, seed=E + 3)
    attn, xres, nw = _vec(E, 80), _vec(E, 81), _norm_w(E, 82)
    y, res1, h = ops.q4nx_o_gemv_ffn(dev(attn), dev(xres), dev(nw), wo_d, wg_d, wu_d, wd_d, return_intermediates=True)
    torch.cuda.synchronize()
    # stage by stage against the float64 oracle, each stage fed the kernel's own previous output
    want1 = oq.gemv_reference(*wo, attn)[0] + bf16_bits_to_f32(xres)
    assert_bf16_close(bits(res1), want1, ulps=1.0, atol=2e-3, what="res1")
    want3 = oq.gemv_reference(*wd, bits(h))[0] + bf16_bits_to_f32(bits(res1))
    assert_bf16_close(bits(y), want3, ulps=1.0, atol=2e-3, what="block y")
    normed = f32_to_bf16_bits(oref.rms_norm_bf16(bits(res1), nw))
    gate = bf16_bits_to_f32(f32_to_bf16_bits(oq.gemv_reference(*wg, normed)[0].astype(np.float32)))
    up = bf16_bits_to_f32(f32_to_bf16_bits(oq.gemv_reference(*wu, normed)[0].astype(np.float32)))
    h_want = bf16_bits_to_f32(f32_to_bf16_bits(oref.silu_tanh_f32(gate) * up))
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), h_want, rtol=0.15, atol=0.5, min_correlation=0.99)
    # end to end against the staged oracle under the reference's gates
    r1, hh, yy = oq.block_staged_reference(wo, wg, wu, wd, attn, xres, nw)
    assert oref.check_outputs(bf16_bits_to_f32(bits(res1)), bf16_bits_to_f32(r1), rtol=0.1, atol=0.05, min_correlation=0.999)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(hh), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(yy), rtol=0.2, atol=2.0, min_correlation=0.99)
    # repeat calls are deterministic and leave the workspace clean
    y2 = ops.q4nx_o_gemv_ffn(dev(attn), dev(xres), dev(nw), wo_d, wg_d, wu_d, wd_d)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y2), bits(y))


def test_decode_block_q4nx_matches_the_oracle_chain(ops):
    """run_decode_block on a Q4NX layer (fused Q|K|V by block concatenation, RoPE + cache append +
    attention, O + FFN) against the oracle's pieces chained on the host."""
    from air_hip import decode, weights
    from helpers import bf16_ulp
    from oracle import decode as odec

    cfg = weights.LlamaConfig(n_layers=1, emb_dim=512, n_heads=8, head_dim=64, n_kv_heads=2, hidden_dim=1024, vocab_size=32)
    E, H, nq, nkv = cfg.emb_dim, cfg.hidden_dim, cfg.n_heads * cfg.head_dim, cfg.kv_dim
    max_seq = 96

    def qw(M, K, seed):   # small weights: w in about [-0.04, 0.04] so that activations stay O(1)
        rng = np.random.default_rng(seed)
        W = (rng.standard_normal((M, K)) * 0.02).astype(np.float32)
        q, sc, mn = oq.requant_q4k(W)
        return q, f32_to_bf16_bits(sc), f32_to_bf16_bits(mn)

    w = {"q": qw(nq, E, 1), "k": qw(nkv, E, 2), "v": qw(nkv, E, 3), "o": qw(E, nq, 4),
         "gate": qw(H, E, 5), "up": qw(H, E, 6), "down": qw(E, H, 7)}
    attn_norm, ffn_norm = _norm_w(E, 8), _norm_w(E, 9)
    layer = decode.prepare_layer_q4nx({k: oq.pack_matrix(*v) for k, v in w.items()}, attn_norm, ffn_norm, cfg)
    assert layer.codec == "q4nx" and layer.wqkv is None and (layer.stream["wqkv"].K, layer.stream["wqkv"].N) == (E, nq + 2 * nkv)
    lut_bits = odec.generate_rope_lut(cfg.head_dim, cfg.rope_base, max_seq)
    lut = decode.generate_rope_lut(cfg, max_seq)
    (kc, vc), = decode.new_kv_cache(cfg, max_seq)
    kc_ref = np.zeros((cfg.n_kv_heads, max_seq, cfg.head_dim), np.uint16)
    vc_ref = np.zeros_like(kc_ref)
    for pos in range(5):
        print(f"q4nx decode block pos={pos}", flush=True)
        x = _vec(E, 500 + pos)
        y = decode.run_decode_block(dev(x), layer, cfg, kc, vc, pos, lut)
        torch.cuda.synchronize()
        q = oq.rms_gemv_reference(w["q"], x, attn_norm)
        k = oq.rms_gemv_reference(w["k"], x, attn_norm)
        v = oq.rms_gemv_reference(w["v"], x, attn_norm)
        q_r = odec.rope_halfsplit(q.reshape(cfg.n_heads, cfg.head_dim), lut_bits[pos]).reshape(-1)
        kc_ref[:, pos] = odec.rope_halfsplit(k.reshape(cfg.n_kv_heads, cfg.head_dim), lut_bits[pos])
        vc_ref[:, pos] = v.reshape(cfg.n_kv_heads, cfg.head_dim)
        attn = odec.decode_attention_cpu(q_r, kc_ref, vc_ref, pos, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim)
        _, _, want = oq.block_staged_reference(w["o"], w["gate"], w["up"], w["down"], attn, x, ffn_norm)
        got_f, want_f = bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(want)
        assert oref.check_outputs(got_f, want_f, rtol=0.2, atol=2.0, min_correlation=0.99)
        assert np.max(np.abs(got_f - want_f)) <= 8 * 2.0**-8 * np.max(np.abs(want_f)), np.max(np.abs(got_f - want_f))
        kd = np.abs(bf16_bits_to_f32(bits(kc)[:, pos]) - bf16_bits_to_f32(kc_ref[:, pos]))
        assert np.all(kd <= 2 * bf16_ulp(bf16_bits_to_f32(kc_ref[:, pos])) + 2e-2), kd.max()
        kc[:, pos] = dev(kc_ref[:, pos])
        vc[:, pos] = dev(vc_ref[:, pos])


def test_prefill_layer_q4nx_agrees_with_decode_steps(ops):
    """A Q4NX layer over a prompt of 70 tokens (run_prefill_layer: the tiled kernel on bf16-rounded weights, causal
    attention over the prompt) against the same tokens fed one at a time through run_decode_block (exact weights, the
    cache growing by one position per step): row m of the prompt pass is step m's output up to the roundings of either
    path, and both leave the same K / V cache."""
    from air_hip import decode, weights

    cfg = weights.LlamaConfig(n_layers=1, emb_dim=512, n_heads=8, head_dim=64, n_kv_heads=2, hidden_dim=1024, vocab_size=32)
    E, H, nq, nkv = cfg.emb_dim, cfg.hidden_dim, cfg.n_heads * cfg.head_dim, cfg.kv_dim
    M, max_seq = 70, 96

    def qw(out, K, seed):
        rng = np.random.default_rng(seed)
        q, sc, mn = oq.requant_q4k((rng.standard_normal((out, K)) * 0.02).astype(np.float32))
        return q, f32_to_bf16_bits(sc), f32_to_bf16_bits(mn)

    w = {"q": qw(nq, E, 11), "k": qw(nkv, E, 12), "v": qw(nkv, E, 13), "o": qw(E, nq, 14),
         "gate": qw(H, E, 15), "up": qw(H, E, 16), "down": qw(E, H, 17)}
    layer = decode.prepare_layer_q4nx({k: oq.pack_matrix(*v) for k, v in w.items()}, _norm_w(E, 18), _norm_w(E, 19), cfg)
    lut = decode.generate_rope_lut(cfg, max_seq)
    rng = np.random.default_rng(20)
    x = dev(f32_to_bf16_bits(rng.standard_normal((M, E)).astype(np.float32)))
    (kc, vc), = decode.new_kv_cache(cfg, max_seq)
    print("q4nx prefill layer, 70 tokens", flush=True)
    y = decode.run_prefill_layer(x, layer, cfg, kc, vc, lut)
    torch.cuda.synchronize()
    (kc2, vc2), = decode.new_kv_cache(cfg, max_seq)
    steps = torch.stack([decode.run_decode_block(x[m].contiguous(), layer, cfg, kc2, vc2, m, lut) for m in range(M)])
    torch.cuda.synchronize()
    err = (y.double() - steps.double()).abs()
    assert float(err.max()) <= 8 * 2.0 ** -8 * float(steps.double().abs().max()), float(err.max())
    for a, b in ((kc, kc2), (vc, vc2)):
        d = (a[:, :M].double() - b[:, :M].double()).abs()
        assert float(d.max()) <= 4 * 2.0 ** -8 * float(b[:, :M].double().abs().max()), float(d.max())


# ---- the same codec in stream order (Q4NX order): whole-K kernels, no workspace ------------------------------------

def _stream_gemv_case(ops, M, K, seed, mode=oq.ADDITIVE, residual=False):
    print(f"q4nx stream gemv M={M} K={K} mode={mode} residual={residual}", flush=True)
    q, s, m = make(M, K, seed)
    rng = np.random.default_rng(seed + 1)
    x = f32_to_bf16_bits(rng.standard_normal((1, K)).astype(np.float32))
    qw, sc, mn = ops.q4nx_repack(dev(oq.pack_matrix(q, s, m)), M, K, mode)
    w = ops.q4nx_repack_stream(qw, sc, mn)
    res = f32_to_bf16_bits(rng.standard_normal(M).astype(np.float32)) if residual else None
    y = ops.q4nx_gemv_stream(dev(x[0]), w, residual=dev(res) if residual else None)
    torch.cuda.synchronize()
    if mode == oq.SUBTRACTIVE:   # the kernel works on the repacked constant term bf16(-s m)
        want = oq.gemv_reference(q, s, bits(mn).T.copy(), x, oq.ADDITIVE)[0]
    else:
        want = oq.gemv_reference(q, s, m, x, mode)[0]
    if residual:
        want = want + bf16_bits_to_f32(res).astype(np.float64)
    got = bits(y)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"q4nx stream gemv M={M} K={K}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, min_correlation=0.999)
    return got, (qw, sc, mn), x


# one block of 16 groups and a short one (K = 256), several blocks with a short last one (K = 14336 = 7 blocks,
# K = 1280 = 10 groups), N from two tiles to the 8B gate width
@pytest.mark.parametrize("M,K", [(32, 256), (2048, 2048), (1024, 4096), (4096, 14336), (3104, 1280), (14336, 4096)])
def test_stream_gemv_shapes(ops, M, K):
    _stream_gemv_case(ops, M, K, seed=M + K)


@pytest.mark.parametrize("mode", [oq.SUBTRACTIVE, oq.Q4_0])
def test_stream_gemv_other_conventions(ops, mode):
    _stream_gemv_case(ops, 2048, 2048, seed=30 + mode, mode=mode)


def test_stream_gemv_with_residual(ops):
    _stream_gemv_case(ops, 4096, 4096, seed=40, residual=False)
    _stream_gemv_case(ops, 1024, 512, seed=41, residual=True)


@pytest.mark.parametrize("rows,M,K,residual", [(2, 512, 1024, False), (16, 512, 1024, True), (7, 64, 256, False), (17, 1024, 512, True),
                                               (40, 512, 1280, False), (16, 14336, 4096, False)])
def test_stream_gemm_rows(ops, rows, M, K, residual):
    """The batched whole-K kernel on the Q4NX order: 2..16 rows per launch, more rows in launches of 16; the tile count of
    N decides how many tiles a workgroup takes (1, 2 or 4)."""
    print(f"q4nx stream gemm rows={rows} M={M} K={K} residual={residual}", flush=True)
    q, s, m = make(M, K, seed=rows + M)
    rng = np.random.default_rng(rows + 1)
    x = f32_to_bf16_bits(rng.standard_normal((rows, K)).astype(np.float32))
    w = ops.q4nx_repack_stream(*ops.q4nx_repack(dev(oq.pack_matrix(q, s, m)), M, K, oq.ADDITIVE))
    res = f32_to_bf16_bits(rng.standard_normal((rows, M)).astype(np.float32)) if residual else None
    y = ops.q4nx_gemm_stream(dev(x), w, residual=dev(res) if residual else None)
    torch.cuda.synchronize()
    want = oq.gemv_reference(q, s, m, x, oq.ADDITIVE)
    if residual:
        want = want + bf16_bits_to_f32(res).astype(np.float64)
    got = bits(y)
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what=f"q4nx stream gemm rows={rows} M={M} K={K}")
    # row r of the batch is the GEMV of row r up to the summation order
    y0 = bits(ops.q4nx_gemv_stream(dev(x[0]), w, residual=dev(res[0]) if residual else None))
    from helpers import bf16_ulp
    a, b = bf16_bits_to_f32(got[0]).astype(np.float64), bf16_bits_to_f32(y0).astype(np.float64)
    assert np.all(np.abs(a - b) <= bf16_ulp(b) + 1e-3)


# From 65 rows on (no residual) the tiled MFMA kernel runs on the Q4NX order: bf16-rounded weights, i.e. the dense
# dequant's values, as the reference's own prompt pass multiplies them (dense bf16 GEMMs on dequantised weights).
# Shapes: N = 64 U with U = 3 (64-column tiles), 8 (128), 13 (256 mixed with 192), 16; K of one block, of two blocks with a
# short one (K = 2304: 18 groups) and of 32 groups; ragged row panels (65, 300) and two full ones (512).
@pytest.mark.parametrize("rows,M,K,wild", [(65, 192, 256, True), (300, 512, 2304, False), (512, 832, 512, True), (130, 1024, 4096, False)])
def test_stream_gemm_tiled(ops, rows, M, K, wild):
    print(f"q4nx tiled stream gemm rows={rows} M={M} K={K} wild={wild}", flush=True)
    q, s, m = make(M, K, seed=rows + M + K, wild=wild)
    rng = np.random.default_rng(rows + 3)
    x = f32_to_bf16_bits(rng.standard_normal((rows, K)).astype(np.float32))
    blocks = oq.pack_matrix(q, s, m)
    w = ops.q4nx_repack_stream(*ops.q4nx_repack(dev(blocks), M, K, oq.ADDITIVE))
    y = ops.q4nx_gemm_stream(dev(x), w)
    torch.cuda.synchronize()
    wd = bf16_bits_to_f32(oq.dequant(blocks, M, K, oq.ADDITIVE)).astype(np.float64)     # [M, K], rounded to bf16
    want = bf16_bits_to_f32(x).astype(np.float64) @ wd.T
    assert_bf16_close(bits(y), want, ulps=1.0, atol=2e-3, what=f"q4nx tiled gemm rows={rows} M={M} K={K}")
    # the first 16 rows through the batched whole-K kernel (exact weights): the two agree up to the weights' rounding
    y16 = bf16_bits_to_f32(bits(ops.q4nx_gemm_stream(dev(x[:16]), w))).astype(np.float64)
    bound = 2.0 ** -8 * (np.abs(bf16_bits_to_f32(x[:16]).astype(np.float64)) @ np.abs(wd.T)) + 2.0 ** -7 * np.abs(y16) + 2e-3
    assert np.all(np.abs(bf16_bits_to_f32(bits(y)[:16]).astype(np.float64) - y16) <= bound)


def test_stream_gemm_tiled_one_hot_rows_are_the_dense_dequant(ops):
    """x = the identity (K rows, one-hot): y[k, :] is row k of W^T, one weight each, so the tiled kernel's output is the
    dense dequant bit for bit; any mix-up of a K-step's scale word with another's shows as a wrong row block of 32."""
    M, K = 320, 256
    q, s, m = make(M, K, seed=77, wild=True)
    blocks = oq.pack_matrix(q, s, m)
    w = ops.q4nx_repack_stream(*ops.q4nx_repack(dev(blocks), M, K, oq.ADDITIVE))
    x = f32_to_bf16_bits(np.eye(K, dtype=np.float32))
    y = ops.q4nx_gemm_stream(dev(x), w)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), oq.dequant(blocks, M, K, oq.ADDITIVE).T)


def _q4_sw(ops, q, s, m):
    M, K = q.shape
    return ops.q4nx_repack_stream(*ops.q4nx_repack(dev(oq.pack_matrix(q, s, m)), M, K, oq.ADDITIVE))


def _q4_dense(q, s, m):
    """[K, out] float64 of the dense dequant's bf16 values."""
    return bf16_bits_to_f32(f32_to_bf16_bits(oq.dequant_values(q, s, m, oq.ADDITIVE))).astype(np.float64).T


@pytest.mark.parametrize("rows,E,H", [(70, 256, 512), (300, 512, 1280)])
def test_prefill_o_ffn_q4nx_stage_by_stage(ops, rows, E, H):
    """The prompt-pass O + FFN block on Q4NX-order weights: every epilogue against the library's own tiled product bit
    for bit (the epilogues work on the bf16 product), every product against float64 on the dense dequant's values."""
    from helpers import bf16_ulp
    print(f"q4nx prefill o+ffn rows={rows} E={E} H={H}", flush=True)
    mats = [make(out, K, seed=rows + i) for i, (out, K) in enumerate(((E, E), (H, E), (H, E), (E, H)))]
    so, sg, su, sd = (_q4_sw(ops, *w) for w in mats)
    do, dg, du, dd = (_q4_dense(*w) for w in mats)
    rng = np.random.default_rng(rows)
    attn = f32_to_bf16_bits(rng.standard_normal((rows, E)).astype(np.float32))
    xres = f32_to_bf16_bits(rng.standard_normal((rows, E)).astype(np.float32))
    nw = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    y, res1, h = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd, return_intermediates=True, codec="q4nx")
    y2 = ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd, codec="q4nx")
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    f = lambda b: bf16_bits_to_f32(b).astype(np.float64)
    add_rounded = lambda prod, add: (prod.float() + add.float()).to(torch.bfloat16)

    def close_sum(got_bits, prod64, add, what):
        want = prod64 + add
        err = np.abs(f(got_bits) - want)
        tol = bf16_ulp(want) + bf16_ulp(prod64) + 2e-3
        assert np.all(err <= tol), f"{what}: {np.max(err - tol)}"

    assert torch.equal(res1.view(torch.int16), add_rounded(ops.q4nx_gemm_stream(dev(attn), so), dev(xres)).view(torch.int16))
    close_sum(bits(res1), f(attn) @ do, f(xres), "res1")
    normed = ops.rms_norm_rows(res1, dev(nw))
    gb, ub = f(bits(ops.q4nx_gemm_stream(normed, sg))), f(bits(ops.q4nx_gemm_stream(normed, su)))
    h_exact = gb / (1.0 + np.exp(-gb)) * ub
    assert np.all(np.abs(f(bits(h)) - h_exact) <= 0.51 * bf16_ulp(h_exact) + 1e-6 * np.abs(h_exact) + 1e-30)
    n64 = f(bits(normed))
    assert_bf16_close(f32_to_bf16_bits(gb.astype(np.float32)), n64 @ dg, ulps=1.0, atol=2e-3, what="gate")
    assert_bf16_close(f32_to_bf16_bits(ub.astype(np.float32)), n64 @ du, ulps=1.0, atol=2e-3, what="up")
    assert torch.equal(y.view(torch.int16), add_rounded(ops.q4nx_gemm_stream(h, sd), res1).view(torch.int16))
    close_sum(bits(y), f(bits(h)) @ dd, f(bits(res1)), "y")
    # an AWQ-order op refuses a Q4NX-order weight instead of reading it with the wrong kernel, and the other way round
    with pytest.raises(ValueError):
        ops.prefill_o_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd)
    with pytest.raises(ValueError):
        ops.w4a16_gemm_stream(dev(attn), so)


@pytest.mark.parametrize("rows,E,nh,nkv,hd,pos0", [(70, 256, 4, 2, 64, 3), (130, 512, 2, 1, 128, 40)])
def test_prefill_rms_qkv_rope_q4nx(ops, rows, E, nh, nkv, hd, pos0):
    """RMSNorm + fused Q|K|V product + half-split RoPE on a Q4NX-order matrix: V is the plain tiled product bit for bit, Q
    and K are the oracle's rotation of that product bit for bit, the product is the float64 one on the dense values."""
    from oracle import decode as odec
    print(f"q4nx prefill qkv rope rows={rows} E={E} heads {nh}/{nkv} hd={hd}", flush=True)
    N = (nh + 2 * nkv) * hd
    q, s, m = make(N, E, seed=rows + N)
    sw = _q4_sw(ops, q, s, m)
    rng = np.random.default_rng(rows + 1)
    x = f32_to_bf16_bits(rng.standard_normal((rows, E)).astype(np.float32))
    nw = f32_to_bf16_bits((rng.standard_normal(E) * 0.1 + 1.0).astype(np.float32))
    lut = odec.generate_rope_lut(hd, 500000.0, pos0 + rows + 2)
    out = ops.prefill_rms_qkv_rope_stream(dev(x), dev(nw), sw, dev(lut), pos0, nh, nkv, hd, codec="q4nx")
    normed = ops.rms_norm_rows(dev(x), dev(nw))
    plain = ops.q4nx_gemm_stream(normed, sw)
    torch.cuda.synchronize()
    got, nq, nk = bits(out), nh * hd, nkv * hd
    assert np.array_equal(got[:, nq + nk:], bits(plain)[:, nq + nk:])
    rows_lut = lut[pos0:pos0 + rows]
    for lo, n in ((0, nh), (nq, nkv)):
        prod = bits(plain)[:, lo:lo + n * hd].reshape(rows * n, hd)
        want = odec.rope_rows(prod, np.repeat(rows_lut, n, axis=0)).reshape(rows, n * hd)
        assert np.array_equal(got[:, lo:lo + n * hd], want)
    assert_bf16_close(bits(plain), bf16_bits_to_f32(bits(normed)).astype(np.float64) @ _q4_dense(q, s, m), ulps=1.0, atol=2e-3,
                      what="q4nx qkv product")


@pytest.mark.parametrize("M,K", [(32, 256), (96, 2304), (1024, 4096)])
def test_stream_device_repack_equals_host_packer(ops, M, K):
    """w4a16_q4nx_repack_stream on the operands of q4nx_repack against the host packer on the same values."""
    from air_hip import awq
    q, s, m = make(M, K, seed=M + K, wild=True)
    qw, sc, mn = ops.q4nx_repack(dev(oq.pack_matrix(q, s, m)), M, K, oq.ADDITIVE)
    w = ops.q4nx_repack_stream(qw, sc, mn)
    torch.cuda.synchronize()
    want = awq.repack_stream_q4nx(q.T.copy(), s.T.copy(), m.T.copy())     # [K, N = M] values
    assert np.array_equal(w.buf.cpu().numpy().view(np.uint32).reshape(want.shape), want)


@pytest.mark.parametrize("mode", [oq.ADDITIVE, oq.SUBTRACTIVE, oq.Q4_0])
@pytest.mark.parametrize("M,K", [(32, 256), (96, 2304), (1024, 4096)])
def test_blocks_to_stream_in_one_pass_equals_the_two_step_repack(ops, M, K, mode):
    """w4a16_q4nx_blocks_to_stream against q4nx_repack followed by w4a16_q4nx_repack_stream: the same buffer, byte for
    byte, in all three value conventions (K = 2304: a short last block of groups; M = 96: an odd number of block rows)."""
    q, s, m = make(M, K, seed=M + K + mode, wild=True)
    blocks = dev(oq.pack_matrix(q, s, m))
    two = ops.q4nx_repack_stream(*ops.q4nx_repack(blocks, M, K, mode))
    one = ops.q4nx_blocks_to_stream(blocks, M, K, mode)
    torch.cuda.synchronize()
    assert (one.K, one.N, one.order) == (two.K, two.N, "q4nx") and torch.equal(one.buf, two.buf)
    with pytest.raises(ValueError):
        ops.q4nx_blocks_to_stream(blocks[:-1], M, K, mode)


def test_stream_gemv_one_hot_x_is_a_dequantised_row(ops):
    """x = e_k picks column k of W[M, K]: s q + min of one 32-column group, a single fp32 fma rounded once: bit for bit
    the dense dequant."""
    M, K = 256, 512
    q, s, m = make(M, K, seed=60, wild=True)
    blocks = dev(oq.pack_matrix(q, s, m))
    w = ops.q4nx_repack_stream(*ops.q4nx_repack(blocks, M, K, oq.ADDITIVE))
    dense = bits(ops.q4nx_dequant(blocks, M, K, oq.ADDITIVE))
    for k in (0, 31, 32, 255, 300, 511):
        x = np.zeros(K, np.uint16)
        x[k] = 0x3F80
        y = bits(ops.q4nx_gemv_stream(dev(x), w))
        assert np.array_equal(y, dense[:, k]), k


@pytest.mark.parametrize("M,K", [(32, 256), (1056, 512), (6144, 4096), (2048, 8192)])
def test_stream_rms_gemv(ops, M, K):
    print(f"q4nx stream rms_gemv M={M} K={K}", flush=True)
    w, wd = _weights(ops, M, K, seed=M + K)
    sw = ops.q4nx_repack_stream(*wd)
    x, nw = _vec(K, 70), _norm_w(K, 71)
    y = ops.q4nx_rms_gemv_stream(dev(x), dev(nw), sw)
    torch.cuda.synchronize()
    want = oq.rms_gemv_reference(w, x, nw)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(want), rtol=0.1, atol=0.05, min_correlation=0.999)
    normed = f32_to_bf16_bits(oref.rms_norm_bf16(x, nw))
    y2 = ops.q4nx_gemv_stream(dev(normed), sw)     # same GEMV without the prologue, fed the oracle's vector
    torch.cuda.synchronize()
    a, b = bf16_bits_to_f32(bits(y)).astype(np.float64), bf16_bits_to_f32(bits(y2)).astype(np.float64)
    from helpers import bf16_ulp
    assert np.all(np.abs(a - b) <= 2 * bf16_ulp(b) + 2e-2), np.abs(a - b).max()


@pytest.mark.parametrize("E,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_stream_o_gemv_ffn_block(ops, E, H):
    print(f"q4nx stream o_gemv_ffn E={E} H={H}", flush=True)
    wo, wo_d = _weights(ops, E, E, seed=E)
    wg, wg_d = _weights(ops, H, E, seed=E + 1)
    wu, wu_d = _weights(ops, H, E, seed=E + 2)
    wd, wd_d = _weights(ops, E, H, seed=E + 3)
    so, sg, su, sd = (ops.q4nx_repack_stream(*t) for t in (wo_d, wg_d, wu_d, wd_d))
    attn, xres, nw = _vec(E, 80), _vec(E, 81), _norm_w(E, 82)
    y, res1, h, sumsq = ops.q4nx_o_gemv_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd, return_intermediates=True,
                                                   return_sumsq=True)
    torch.cuda.synchronize()
    want1 = oq.gemv_reference(*wo, attn)[0] + bf16_bits_to_f32(xres)
    assert_bf16_close(bits(res1), want1, ulps=1.0, atol=2e-3, what="res1")
    want3 = oq.gemv_reference(*wd, bits(h))[0] + bf16_bits_to_f32(bits(res1))
    assert_bf16_close(bits(y), want3, ulps=1.0, atol=2e-3, what="block y")
    normed = f32_to_bf16_bits(oref.rms_norm_bf16(bits(res1), nw))
    gate = bf16_bits_to_f32(f32_to_bf16_bits(oq.gemv_reference(*wg, normed)[0].astype(np.float32)))
    up = bf16_bits_to_f32(f32_to_bf16_bits(oq.gemv_reference(*wu, normed)[0].astype(np.float32)))
    h_want = bf16_bits_to_f32(f32_to_bf16_bits(oref.silu_tanh_f32(gate) * up))
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), h_want, rtol=0.15, atol=0.5, min_correlation=0.99)
    r1, hh, yy = oq.block_staged_reference(wo, wg, wu, wd, attn, xres, nw)
    assert oref.check_outputs(bf16_bits_to_f32(bits(res1)), bf16_bits_to_f32(r1), rtol=0.1, atol=0.05, min_correlation=0.999)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(hh), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(yy), rtol=0.2, atol=2.0, min_correlation=0.99)
    # the sums of squares the next layer's norm will use are those of the rounded outputs, 16 columns at a time
    yf = bf16_bits_to_f32(bits(y)).astype(np.float64)
    assert np.allclose(sumsq.cpu().numpy(), (yf ** 2).reshape(-1, 16).sum(axis=1), rtol=1e-5)
    y2 = ops.q4nx_o_gemv_ffn_stream(dev(attn), dev(xres), dev(nw), so, sg, su, sd)
    torch.cuda.synchronize()
    assert np.array_equal(bits(y2), bits(y))


def test_stream_launches_replay_from_a_hip_graph(ops):
    """RMSNorm + Q|K|V GEMV, the O + FFN block and the batched kernel (which raises its LDS limit by a function
    attribute at launch) on Q4NX-order weights, captured in one HIP graph: every replay, with eager work and
    synchronisations in between, equals the eager results bit for bit."""
    E, H = 512, 1024
    print(f"q4nx stream graph E={E} H={H}", flush=True)
    sw = [ops.q4nx_repack_stream(*_weights(ops, M, K, seed=900 + i)[1]) for i, (M, K) in enumerate([(3 * E, E), (E, E), (H, E), (H, E), (E, H)])]
    wqkv, so, sg, su, sd = sw
    nw_a, nw_f = dev(_norm_w(E, 910)), dev(_norm_w(E, 911))
    rng = np.random.default_rng(912)
    vecs = [dev(f32_to_bf16_bits(rng.standard_normal((3, E)).astype(np.float32))) for _ in range(3)]   # x, attn, residual per replay
    rows = [dev(f32_to_bf16_bits(rng.standard_normal((16, E)).astype(np.float32))) for _ in range(3)]
    cur_v, cur_r = vecs[0].clone(), rows[0].clone()

    def step(v, r):
        qkv = ops.q4nx_rms_gemv_stream(v[0], nw_a, wqkv)
        y = ops.q4nx_o_gemv_ffn_stream(v[1], v[2], nw_f, so, sg, su, sd)
        return qkv, y, ops.q4nx_gemm_stream(r, so)

    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        step(cur_v, cur_r)   # warm-up: scratch buffers and the function attribute outside the graph
        st.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            outs = step(cur_v, cur_r)
        for j in range(3):
            cur_v.copy_(vecs[j])
            cur_r.copy_(rows[j])
            g.replay()
            st.synchronize()
            want = step(vecs[j], rows[j])
            st.synchronize()
            for name, a, b in zip(("qkv", "block", "gemm16"), outs, want):
                assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (name, j)


def test_stream_entry_points_reject_bad_arguments(ops):
    from air_hip import _lib
    lib = _lib.load_library()
    P = torch.zeros(1 << 16, dtype=torch.int32, device="cuda").data_ptr()
    assert lib.w4a16_q4nx_stream_bytes(256, 24) == 0 and lib.w4a16_q4nx_stream_bytes(192, 32) == 0
    assert lib.w4a16_q4nx_stream_bytes(256, 32) == 2 * (4 + 2) * 1024
    assert lib.w4a16_q4nx_repack_stream(P, P, None, P, 256, 32, None) == _lib.ERR_NULL
    assert lib.w4a16_q4nx_repack_stream(P, P, P, P, 200, 32, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_gemv_stream_bf16(P, P, None, P, 256, 40, None) == _lib.ERR_SHAPE
    assert lib.w4a16_q4nx_gemv_stream_bf16(P, None, None, P, 256, 32, None) == _lib.ERR_NULL
    assert lib.w4a16_q4nx_gemv_stream_bf16(P + 2, P, None, P, 256, 32, None) == _lib.ERR_ALIGN
    assert lib.w4a16_q4nx_rms_gemv_stream_bf16(P, None, 0, None, 1e-5, P, P, 256, 32, None) == _lib.ERR_NULL
    ws = lib.w4a16_block_stream_workspace_bytes(256, 256)
    assert lib.w4a16_q4nx_o_gemv_ffn_stream_bf16(P, P, P, 1e-5, P, P, P, P, P, None, None, None, 256, 256, P, ws - 1, None) == _lib.ERR_WORKSPACE
