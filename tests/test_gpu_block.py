"""GPU parity of the decode-block stages: GEMV + residual, RMSNorm prologue, the RMSNorm +
gate/up + SwiGLU kernel and the three-stage O + FFN block, through the C ABI.

Tolerances.  A stage output is one bf16 rounding of an fp32 sum: 1 bf16 ulp of the float64
oracle + 2e-3 absolute.  The RMSNorm prologue rounds n = (x * rstd) * w to bf16; the kernel's
fp32 rstd may differ from the oracle's by an ulp of fp32, which can flip that rounding in a
few elements.  So the kernel's normalised vector itself is checked against the oracle's
(identity-like weights make the GEMV return it), and GEMV results after a prologue are checked against the oracle with
that flip propagated through |W|.  End-to-end results also pass the reference's own gates."""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close, bf16_ulp, dense_f64, make_awq, make_x
from oracle import awq as oawq, reference as oref
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


@pytest.mark.parametrize("K,N", [(128, 32), (512, 1056), (4096, 4096), (8192, 2048)])
def test_gemv_add(ops, K, N):
    print(f"gemv_add K={K} N={N}", flush=True)
    qw, qz, s = make_awq(K, N, seed=K + N)
    x = make_x((K,), seed=7)
    r = make_x((N,), seed=8)
    y = ops.w4a16_gemv_add(dev(x), dev(qw), dev(qz), dev(s), dev(r))
    torch.cuda.synchronize()
    want = bf16_bits_to_f32(x).astype(np.float64) @ dense_f64(qw, qz, s) + bf16_bits_to_f32(r)
    assert_bf16_close(bits(y), want, ulps=1.0, atol=2e-3, what="gemv_add")
    l1 = oawq.repack_hf_awq_linear(qw, qz, s, 128)
    ref = oref.matvec_add_cpu_reference(*l1, x, r)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(ref), rtol=0.1, atol=0.05,
                              min_correlation=0.999)


def test_gemv_add_zero_weights_returns_the_residual_bit_exactly(ops):
    print("gemv_add q == z", flush=True)
    K, N = 256, 544
    rng = np.random.default_rng(3)
    z = rng.integers(0, 16, size=(K // 128, N), dtype=np.uint8)
    q = np.repeat(z, 128, axis=0)                    # q == z everywhere: W = 0
    s = f32_to_bf16_bits(np.full((K // 128, N), 0.01, np.float32))
    r = make_x((N,), seed=4)
    y = ops.w4a16_gemv_add(dev(make_x((K,), seed=5)), dev(oawq.pack_awq_int32(q)), dev(oawq.pack_awq_int32(z)),
                           dev(s), dev(r))
    torch.cuda.synchronize()
    assert np.array_equal(bits(y), r)


def _rms_vectors(K, seed):
    x = make_x((K,), seed=seed)
    w = make_norm_w(K, seed + 1)
    return x, w, oref.rms_norm_bf16(x, w).astype(np.float64)


@pytest.mark.parametrize("K,N", [(128, 32), (512, 1056), (2048, 4096), (4096, 2048)])
def test_rms_gemv(ops, K, N):
    print(f"rms_gemv K={K} N={N}", flush=True)
    qw, qz, s = make_awq(K, N, seed=K + N + 1)
    x, w, normed = _rms_vectors(K, seed=11)
    y = ops.w4a16_rms_gemv(dev(x), dev(w), dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    W = dense_f64(qw, qz, s)
    want = normed @ W
    # the kernel's n may differ from the oracle's by one bf16 ulp in a few elements
    slack = (bf16_ulp(normed) * 0.02) @ np.abs(W)     # at most ~2 % of elements flip
    got = bf16_bits_to_f32(bits(y)).astype(np.float64)
    assert np.all(np.abs(got - want) <= bf16_ulp(want) + 2e-3 + slack), np.abs(got - want).max()


def test_rms_gemv_recovers_the_normalised_vector(ops):
    """W = identity-like (q - z = 1 on the diagonal, 0 elsewhere, s = 1): y is the normalised
    vector, up to the kernel's fp32 cancellation slack (it sums (128 + q) * n and subtracts
    (128 + z) * sum n) and the one-ulp flips of the prologue's rounding."""
    print("rms_gemv identity", flush=True)
    K = N = 512
    z = np.full((K // 128, N), 7, np.uint8)
    q = np.full((K, N), 7, np.uint8)
    q[np.arange(K), np.arange(N)] = 8
    s = np.full((K // 128, N), 0x3F80, np.uint16)
    x, w, normed = _rms_vectors(K, seed=21)
    y = ops.w4a16_rms_gemv(dev(x), dev(w), dev(oawq.pack_awq_int32(q)), dev(oawq.pack_awq_int32(z)), dev(s))
    torch.cuda.synchronize()
    assert_bf16_close(bits(y), normed, ulps=1.0, atol=2e-3, what="normalised vector")


def test_rms_gemv_is_invariant_to_power_of_two_scaling_of_x(ops):
    """With eps = 0, rms_norm(4x) == rms_norm(x) exactly (scaling by 4 is exact in every step)."""
    print("rms_gemv scale invariance", flush=True)
    K, N = 1024, 512
    qw, qz, s = make_awq(K, N, seed=31)
    x = make_x((K,), seed=32)
    x4 = f32_to_bf16_bits(bf16_bits_to_f32(x) * 4.0)
    w = make_norm_w(K, 33)
    a = ops.w4a16_rms_gemv(dev(x), dev(w), dev(qw), dev(qz), dev(s), eps=0.0)
    b = ops.w4a16_rms_gemv(dev(x4), dev(w), dev(qw), dev(qz), dev(s), eps=0.0)
    torch.cuda.synchronize()
    assert np.array_equal(bits(a), bits(b))


@pytest.mark.parametrize("K,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_rms_swiglu(ops, K, H):
    print(f"rms_swiglu K={K} H={H}", flush=True)
    g = make_awq(K, H, seed=K + 1)
    u = make_awq(K, H, seed=K + 2)
    x, w, normed = _rms_vectors(K, seed=K + 3)
    h = ops.w4a16_rms_swiglu(dev(x), dev(w), tuple(map(dev, g)), tuple(map(dev, u)))
    torch.cuda.synchronize()
    a_q, a_s, a_z = oref.interleave_gate_up(oawq.repack_hf_awq_linear(*g, 128), oawq.repack_hf_awq_linear(*u, 128))
    ref = oref.swiglu_rms_cpu_reference(a_q, a_s, a_z, x, w)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(ref), rtol=0.15, atol=0.5,
                              min_correlation=0.99)
    # tighter: the same kernel without the prologue, fed the oracle's normalised vector, must agree with
    # the fused kernel except where a one-ulp flip of n moved a result
    h2 = ops.w4a16_swiglu(dev(f32_to_bf16_bits(normed.astype(np.float32))), tuple(map(dev, g)), tuple(map(dev, u)))
    torch.cuda.synchronize()
    a = bf16_bits_to_f32(bits(h)).astype(np.float64)
    b = bf16_bits_to_f32(bits(h2)).astype(np.float64)
    assert np.all(np.abs(a - b) <= 4 * bf16_ulp(b) + 2e-2), np.abs(a - b).max()
    print(f"  fused vs unfused bit mismatch: {np.mean(bits(h) != bits(h2)):.4f}", flush=True)


@pytest.mark.parametrize("E,H", [(256, 512), (2048, 8192), (4096, 14336)])
def test_o_gemv_ffn_block(ops, E, H):
    print(f"o_gemv_ffn E={E} H={H}", flush=True)
    wo = make_awq(E, E, seed=E)
    g = make_awq(E, H, seed=E + 1)
    u = make_awq(E, H, seed=E + 2)
    d = make_awq(H, E, seed=E + 3)
    attn = make_x((E,), seed=E + 4)
    xres = make_x((E,), seed=E + 5)
    w = make_norm_w(E, E + 6)
    dv = lambda t: tuple(map(dev, t))
    y, res1, h = ops.o_gemv_ffn(dev(attn), dev(xres), dev(w), dv(wo), dv(g), dv(u), dv(d), return_intermediates=True)
    torch.cuda.synchronize()
    # stage by stage against the float64 oracle, each stage fed the kernel's own previous output
    want1 = bf16_bits_to_f32(attn).astype(np.float64) @ dense_f64(*wo) + bf16_bits_to_f32(xres)
    assert_bf16_close(bits(res1), want1, ulps=1.0, atol=2e-3, what="res1")
    h_alone = ops.w4a16_rms_swiglu(res1, dev(w), dv(g), dv(u))
    torch.cuda.synchronize()
    assert np.array_equal(bits(h), bits(h_alone))
    want3 = bf16_bits_to_f32(bits(h)).astype(np.float64) @ dense_f64(*d) + bf16_bits_to_f32(bits(res1))
    assert_bf16_close(bits(y), want3, ulps=1.0, atol=2e-3, what="block y")
    # end to end under the reference's gate, against both references of the block
    l1 = lambda t: oawq.repack_hf_awq_linear(*t, 128)
    r1, hh, yy = oref.o_gemv_ffn_staged_reference(l1(wo), l1(g), l1(u), l1(d), attn, xres, w)
    assert oref.check_outputs(bf16_bits_to_f32(bits(res1)), bf16_bits_to_f32(r1), rtol=0.1, atol=0.05, min_correlation=0.999)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(hh), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(yy), rtol=0.2, atol=2.0, min_correlation=0.99)
    dq = lambda t: np.ascontiguousarray(oawq.dequant_to_bf16(*t, 128).T)
    whole = oref.o_gemv_ffn_int4_reference(dq(wo), attn, xres, w, dq(g), dq(u), dq(d))
    # (its weights are bf16-rounded and its intermediates are not: with these wide synthetic weights
    # that moves single elements by more than the gate's atol, so the distance is bounded in norm;
    # the example test runs the gate itself on the reference's own weight distribution)
    yf, wf = bf16_bits_to_f32(bits(y)).astype(np.float64), bf16_bits_to_f32(whole).astype(np.float64)
    assert np.linalg.norm(yf - wf) <= 0.02 * np.linalg.norm(wf)
    assert np.corrcoef(yf, wf)[0, 1] >= 0.999


def test_block_repeat_calls_are_deterministic(ops):
    print("block repeat", flush=True)
    E, H = 2048, 8192
    dv = lambda t: tuple(map(dev, t))
    wo, g, u, d = dv(make_awq(E, E, seed=1)), dv(make_awq(E, H, seed=2)), dv(make_awq(E, H, seed=3)), dv(make_awq(H, E, seed=4))
    attn, xres, w = dev(make_x((E,), seed=5)), dev(make_x((E,), seed=6)), dev(make_norm_w(E, 7))
    first = bits(ops.o_gemv_ffn(attn, xres, w, wo, g, u, d))
    for _ in range(4):
        assert np.array_equal(bits(ops.o_gemv_ffn(attn, xres, w, wo, g, u, d)), first)
