"""GPU parity of the decode path on stream-order weights (through the C ABI): RMSNorm prologue, RMSNorm + gate / up +
SwiGLU, the FFN, the three-stage O + FFN block, the chained sum of squares and a decode block over several tokens.

Tolerances as for the checkpoint-layout entry points: a stage output is one bf16 rounding of an fp32 sum (1 bf16 ulp of
the float64 oracle + 2e-3); the RMSNorm prologue's fp32 rstd may differ from the oracle's by an ulp of fp32, which can
flip the bf16 rounding of a few normalised elements, so results behind a prologue carry that flip propagated through
|W|, and the normalised vector itself is recovered through identity-like weights.  End-to-end results also pass the
reference's own gates."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close, bf16_ulp, dense_f64, make_awq, make_x
from oracle import awq as oawq, decode as odec, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def make_norm_w(K, seed):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits((rng.standard_normal(K) * 0.1 + 1.0).astype(np.float32))


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


def sw(ops, t):
    return ops.repack_stream(*map(dev, t))


def _rms_vectors(K, seed):
    x = make_x((K,), seed=seed)
    w = make_norm_w(K, seed + 1)
    return x, w, oref.rms_norm_bf16(x, w).astype(np.float64)


@pytest.mark.parametrize("K,N", [(128, 32), (512, 1056), (2048, 4096), (4096, 2048), (128 * 19, 48)])
def test_rms_gemv_stream(ops, K, N):
    print(f"rms_gemv stream K={K} N={N}", flush=True)
    t = make_awq(K, N, seed=K + N + 1)
    x, w, normed = _rms_vectors(K, seed=11)
    y = ops.w4a16_rms_gemv_stream(dev(x), dev(w), sw(ops, t))
    torch.cuda.synchronize()
    W = dense_f64(*t)
    want = normed @ W
    slack = (bf16_ulp(normed) * 0.02) @ np.abs(W)     # at most ~2 % of the normalised elements flip by one ulp
    got = bf16_bits_to_f32(bits(y)).astype(np.float64)
    assert np.all(np.abs(got - want) <= bf16_ulp(want) + 2e-3 + slack), np.abs(got - want).max()


def test_rms_gemv_stream_recovers_the_normalised_vector(ops):
    """W = identity-like (q - z = 1 on the diagonal, 0 elsewhere, s = 1): y is the normalised vector."""
    K = N = 512
    z = np.full((K // 128, N), 7, np.uint8)
    q = np.full((K, N), 7, np.uint8)
    q[np.arange(K), np.arange(N)] = 8
    s = np.full((K // 128, N), 0x3F80, np.uint16)
    x, w, normed = _rms_vectors(K, seed=21)
    y = ops.w4a16_rms_gemv_stream(dev(x), dev(w), sw(ops, (oawq.pack_awq_int32(q), oawq.pack_awq_int32(z), s)))
    torch.cuda.synchronize()
    assert_bf16_close(bits(y), normed, ulps=1.0, atol=2e-3, what="normalised vector")


def test_rms_gemv_stream_is_invariant_to_power_of_two_scaling_of_x(ops):
    K, N = 1024, 512
    t = make_awq(K, N, seed=31)
    x = make_x((K,), seed=32)
    x4 = f32_to_bf16_bits(bf16_bits_to_f32(x) * 4.0)
    w = make_norm_w(K, 33)
    wt = sw(ops, t)
    a = ops.w4a16_rms_gemv_stream(dev(x), dev(w), wt, eps=0.0)
    b = ops.w4a16_rms_gemv_stream(dev(x4), dev(w), wt, eps=0.0)
    torch.cuda.synchronize()
    assert np.array_equal(bits(a), bits(b))


def test_rms_gemv_stream_takes_the_sum_of_squares_from_its_producer(ops):
    """A GEMV + residual leaves sum(y^2) per 16 columns; the next RMSNorm + GEMV takes those pieces instead of walking
    its input: same normalised vector up to the summation order of the mean."""
    E, N = 2048, 3072
    wo, wq = make_awq(E, E, seed=41), make_awq(E, N, seed=42)
    w_norm = make_norm_w(E, 43)
    y, sumsq = ops.o_gemv_ffn_stream(dev(make_x((E,), seed=44)), dev(make_x((E,), seed=45)), dev(make_norm_w(E, 46)),
                                     sw(ops, wo), sw(ops, make_awq(E, 1024, seed=47)), sw(ops, make_awq(E, 1024, seed=48)),
                                     sw(ops, make_awq(1024, E, seed=49)), return_sumsq=True)
    torch.cuda.synchronize()
    yf = bf16_bits_to_f32(bits(y)).astype(np.float64)
    want_pieces = (yf ** 2).reshape(E // 16, 16).sum(axis=1)
    assert np.allclose(sumsq.cpu().numpy(), want_pieces, rtol=1e-5, atol=1e-6)
    wt = sw(ops, wq)
    a = ops.w4a16_rms_gemv_stream(y, dev(w_norm), wt)
    b = ops.w4a16_rms_gemv_stream(y, dev(w_norm), wt, x_sumsq=sumsq)
    torch.cuda.synchronize()
    af, bf = bf16_bits_to_f32(bits(a)).astype(np.float64), bf16_bits_to_f32(bits(b)).astype(np.float64)
    normed = oref.rms_norm_bf16(bits(y), w_norm).astype(np.float64)
    slack = (bf16_ulp(normed) * 0.02) @ np.abs(dense_f64(*wq))
    assert np.all(np.abs(af - bf) <= 2 * bf16_ulp(af) + 2e-3 + 2 * slack), np.abs(af - bf).max()


@pytest.mark.parametrize("K,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_rms_swiglu_stream(ops, K, H):
    print(f"rms_swiglu stream K={K} H={H}", flush=True)
    g, u = make_awq(K, H, seed=K + 1), make_awq(K, H, seed=K + 2)
    x, w, normed = _rms_vectors(K, seed=K + 3)
    gs, us = sw(ops, g), sw(ops, u)
    h = ops.w4a16_rms_swiglu_stream(dev(x), dev(w), gs, us)
    torch.cuda.synchronize()
    a_q, a_s, a_z = oref.interleave_gate_up(oawq.repack_hf_awq_linear(*g, 128), oawq.repack_hf_awq_linear(*u, 128))
    ref = oref.swiglu_rms_cpu_reference(a_q, a_s, a_z, x, w)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(ref), rtol=0.15, atol=0.5, min_correlation=0.99)
    # the same kernel without the prologue, fed the oracle's normalised vector
    h2 = ops.w4a16_swiglu_stream(dev(f32_to_bf16_bits(normed.astype(np.float32))), gs, us)
    torch.cuda.synchronize()
    a, b = bf16_bits_to_f32(bits(h)).astype(np.float64), bf16_bits_to_f32(bits(h2)).astype(np.float64)
    assert np.all(np.abs(a - b) <= 4 * bf16_ulp(b) + 2e-2), np.abs(a - b).max()


def _ffn_case(ops, K, H, seed):
    print(f"ffn stream K={K} H={H}", flush=True)
    g, u, d = make_awq(K, H, seed=seed), make_awq(K, H, seed=seed + 1), make_awq(H, K, seed=seed + 2)
    x = make_x((K,), seed=seed + 3)
    y, h = ops.ffn_swiglu_stream(dev(x), sw(ops, g), sw(ops, u), sw(ops, d), return_h=True)
    torch.cuda.synchronize()
    xf = bf16_bits_to_f32(x).astype(np.float64)
    gb = bf16_bits_to_f32(f32_to_bf16_bits((xf @ dense_f64(*g)).astype(np.float32)))
    ub = bf16_bits_to_f32(f32_to_bf16_bits((xf @ dense_f64(*u)).astype(np.float32)))
    h_want = oref.silu_tanh_f32(gb).astype(np.float64) * ub
    assert_bf16_close(bits(h), h_want, ulps=4.0, atol=2e-3, what="ffn h")
    y_want = bf16_bits_to_f32(bits(h)).astype(np.float64) @ dense_f64(*d)
    assert_bf16_close(bits(y), y_want, ulps=1.0, atol=2e-3, what="ffn y")
    l1 = lambda t: oawq.repack_hf_awq_linear(*t, 128)
    h_ref, y_ref = oref.ffn_swiglu_reference(l1(g), l1(u), l1(d), x)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(h_ref), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(y_ref), rtol=0.2, atol=2.0, min_correlation=0.99)


def test_ffn_stream_small(ops):
    _ffn_case(ops, 256, 512, seed=20)
    _ffn_case(ops, 1024, 2048 + 128, seed=30)


def test_ffn_stream_config4(ops):
    _ffn_case(ops, 4096, 14336, seed=40)


@pytest.mark.parametrize("E,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_o_gemv_ffn_stream_block(ops, E, H):
    print(f"o_gemv_ffn stream E={E} H={H}", flush=True)
    wo, g, u, d = make_awq(E, E, seed=E), make_awq(E, H, seed=E + 1), make_awq(E, H, seed=E + 2), make_awq(H, E, seed=E + 3)
    attn, xres, w = make_x((E,), seed=E + 4), make_x((E,), seed=E + 5), make_norm_w(E, E + 6)
    wos, gs, us, ds = sw(ops, wo), sw(ops, g), sw(ops, u), sw(ops, d)
    y, res1, h = ops.o_gemv_ffn_stream(dev(attn), dev(xres), dev(w), wos, gs, us, ds, return_intermediates=True)
    torch.cuda.synchronize()
    want1 = bf16_bits_to_f32(attn).astype(np.float64) @ dense_f64(*wo) + bf16_bits_to_f32(xres)
    assert_bf16_close(bits(res1), want1, ulps=1.0, atol=2e-3, what="res1")
    # stage 2 alone (walking res1 for the mean instead of taking the pieces) agrees up to one-ulp flips
    h_alone = ops.w4a16_rms_swiglu_stream(res1, dev(w), gs, us)
    torch.cuda.synchronize()
    a, b = bf16_bits_to_f32(bits(h)).astype(np.float64), bf16_bits_to_f32(bits(h_alone)).astype(np.float64)
    assert np.all(np.abs(a - b) <= 4 * bf16_ulp(b) + 2e-2), np.abs(a - b).max()
    want3 = bf16_bits_to_f32(bits(h)).astype(np.float64) @ dense_f64(*d) + bf16_bits_to_f32(bits(res1))
    assert_bf16_close(bits(y), want3, ulps=1.0, atol=2e-3, what="block y")
    l1 = lambda t: oawq.repack_hf_awq_linear(*t, 128)
    r1, hh, yy = oref.o_gemv_ffn_staged_reference(l1(wo), l1(g), l1(u), l1(d), attn, xres, w)
    assert oref.check_outputs(bf16_bits_to_f32(bits(res1)), bf16_bits_to_f32(r1), rtol=0.1, atol=0.05, min_correlation=0.999)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(hh), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(yy), rtol=0.2, atol=2.0, min_correlation=0.99)
    # repeat calls are deterministic (fixed summation order, no state between calls)
    for _ in range(3):
        assert np.array_equal(bits(ops.o_gemv_ffn_stream(dev(attn), dev(xres), dev(w), wos, gs, us, ds)), bits(y))


def test_stream_block_agrees_with_the_checkpoint_layout_block(ops):
    """Both layouts compute the same sums in different orders: outputs agree to a few bf16 ulps."""
    E, H = 2048, 8192
    wo, g, u, d = make_awq(E, E, seed=1), make_awq(E, H, seed=2), make_awq(E, H, seed=3), make_awq(H, E, seed=4)
    attn, xres, w = dev(make_x((E,), seed=5)), dev(make_x((E,), seed=6)), dev(make_norm_w(E, 7))
    dv = lambda t: tuple(map(dev, t))
    a = bf16_bits_to_f32(bits(ops.o_gemv_ffn(attn, xres, w, dv(wo), dv(g), dv(u), dv(d)))).astype(np.float64)
    b = bf16_bits_to_f32(bits(ops.o_gemv_ffn_stream(attn, xres, w, sw(ops, wo), sw(ops, g), sw(ops, u), sw(ops, d)))).astype(np.float64)
    assert np.max(np.abs(a - b)) <= 8 * 2.0**-8 * np.max(np.abs(a))
