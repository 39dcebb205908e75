"""GPU parity: HIP kernels (through the C ABI) against the CPU oracle.

Tolerances.  Dequant: bit-exact.  GEMV / GEMM / FFN: the result is one bf16
rounding of an fp32-accumulated sum, so it must lie within 1 bf16 ulp of the
float64 oracle value plus 2e-3 absolute (cancellation slack for |y| << sum|terms|),
and must also pass the reference's own gate (rtol 0.1, atol 0.05, r >= 0.999).
"""
import numpy as np
import pytest
import torch

from helpers import assert_bf16_close, dense_f64, make_awq, make_x
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


@pytest.fixture(scope="module")
def ops():
    from air_hip import ops
    return ops


@pytest.mark.parametrize("K,N", [(128, 8), (256, 64), (384, 40), (128, 2056), (1024, 1024)])
def test_dequant_bit_exact_small(ops, K, N):
    print(f"dequant K={K} N={N}", flush=True)
    qw, qz, s = make_awq(K, N, seed=K + N)
    out = ops.awq_dequant(dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oawq.dequant_to_bf16(qw, qz, s, 128))


def test_dequant_bit_exact_config0(ops):
    print("dequant config0", flush=True)
    K = N = 4096
    qw, qz, s = make_awq(K, N, seed=0)
    out = ops.awq_dequant(dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oawq.dequant_to_bf16(qw, qz, s, 128))


def test_dequant_negative_and_extreme_scales(ops):
    print("dequant extreme scales", flush=True)
    K, N = 256, 64
    qw, qz, _ = make_awq(K, N, seed=5)
    rng = np.random.default_rng(6)
    s = rng.integers(0, 65536, size=(K // 128, N)).astype(np.uint16)
    s[(s & 0x7F80) == 0x7F80] = 0x3C00          # no inf/nan scales
    out = ops.awq_dequant(dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    assert np.array_equal(bits(out), oawq.dequant_to_bf16(qw, qz, s, 128))


def _gemm_case(ops, M, K, N, seed, ulps=1.0, atol=2e-3):
    print(f"gemm M={M} K={K} N={N} seed={seed}", flush=True)
    qw, qz, s = make_awq(K, N, seed=seed)
    x = make_x((M, K), seed=seed + 1)
    y = ops.w4a16_gemm(dev(x), dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    got = bits(y)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    want = xf @ dense_f64(qw, qz, s, rounded=(M > 96))   # M <= 96 streams exact weights, larger M multiplies bf16-rounded ones
    assert_bf16_close(got, want, ulps=ulps, atol=atol, what=f"gemm M={M} K={K} N={N}")
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want.astype(np.float32))),
                              rtol=0.1, atol=0.05, min_correlation=0.999 if want.size > 8 else None)
    return got, want


@pytest.mark.parametrize("K,N", [(128, 32), (256, 544), (512, 1056), (1024, 512), (4096, 4096), (2048, 8192)])
def test_gemv_small(ops, K, N):
    _gemm_case(ops, 1, K, N, seed=K + N)


def test_gemv_config1(ops):
    _gemm_case(ops, 1, 4096, 11008, seed=1)


def test_gemv_one_hot_x_is_a_dequantised_row(ops):
    print("gemv one-hot", flush=True)
    K, N = 512, 1024
    qw, qz, s = make_awq(K, N, seed=3)
    w = oawq.dequant_to_bf16(qw, qz, s, 128)
    for k0 in (0, 1, 127, 128, 300, 511):
        x = np.zeros(K, np.uint16)
        x[k0] = 0x3F80
        y = ops.w4a16_gemv(dev(x), dev(qw), dev(qz), dev(s))
        torch.cuda.synchronize()
        assert np.array_equal(bits(y), w[k0]), k0


@pytest.mark.parametrize("ksplit", [1, 3, 5, 7])
def test_gemv_uneven_k_slices(ops, ksplit):
    """K-slices whose sizes differ by one unit (K = 1024 + 128: 9 units over `ksplit` workgroups)."""
    ops.tune("gemv_ksplit", ksplit)
    try:
        _gemm_case(ops, 1, 1152, 544, seed=60 + ksplit)
        _gemm_case(ops, 7, 1152, 544, seed=70 + ksplit)
    finally:
        ops.tune("gemv_ksplit", 0)


def test_gemv_grid_larger_than_the_chip(ops):
    """2052 workgroups (513 column tiles x 4 K-slices, ragged last tile) on 256 CUs: reducers are
    dispatched after their producers, so a grid of several rounds still completes."""
    _gemm_case(ops, 1, 4096, 131072 + 96, seed=77)


def test_one_workspace_serves_interleaved_shapes(ops):
    """Every launch leaves the partial slots it used empty again, so launches of different shapes
    (different slot maps) can alternate on one workspace without re-initialising it."""
    print("interleaved shapes on one workspace", flush=True)
    cases = []
    for M, K, N, seed in [(1, 4096, 11008, 1), (16, 1024, 4128, 2), (1, 14336, 4096, 3), (5, 512, 32, 4), (1, 2048, 2048, 5)]:
        qw, qz, s = make_awq(K, N, seed=seed)
        args = (dev(make_x((M, K), seed=seed + 10)), dev(qw), dev(qz), dev(s))
        cases.append((args, bits(ops.w4a16_gemm(*args))))
    g = make_awq(1024, 2048, seed=6), make_awq(1024, 2048, seed=7), make_awq(2048, 1024, seed=8)
    gd = [tuple(map(dev, t)) for t in g]
    xf = dev(make_x((1024,), seed=9))
    ffn_first = bits(ops.ffn_swiglu(xf, *gd))
    for it in range(40):
        for args, first in cases:
            assert np.array_equal(bits(ops.w4a16_gemm(*args)), first), it
        assert np.array_equal(bits(ops.ffn_swiglu(xf, *gd)), ffn_first), it


def test_gemv_repeat_calls_are_deterministic_and_workspace_is_reusable(ops):
    print("gemv repeat", flush=True)
    K, N = 4096, 11008
    qw, qz, s = make_awq(K, N, seed=9)
    x = make_x((K,), seed=10)
    dq, dz, ds, dx = dev(qw), dev(qz), dev(s), dev(x)
    first = bits(ops.w4a16_gemv(dx, dq, dz, ds))
    for _ in range(5):
        assert np.array_equal(bits(ops.w4a16_gemv(dx, dq, dz, ds)), first)


@pytest.mark.parametrize("M", [2, 3, 4, 5, 8, 13, 16, 17, 40, 96])
def test_small_m_gemm(ops, M):
    _gemm_case(ops, M, 1024, 1056, seed=M)


def test_gemm_config2(ops):
    _gemm_case(ops, 16, 4096, 14336, seed=2)


@pytest.mark.parametrize("M,K,N", [(97, 128, 32), (100, 256, 128), (130, 512, 544), (200, 1024, 1056), (256, 4096, 512)])
def test_prefill_gemm_small(ops, M, K, N):
    _gemm_case(ops, M, K, N, seed=M + K + N)


@pytest.mark.parametrize("M,K,N", [(17, 128, 32), (64, 256, 128)])
def test_prefill_kernel_at_small_m(ops, M, K, N):
    """The tiled kernel itself on tiles that are mostly padding (the boundary to the streaming
    kernel lowered to 16)."""
    ops.tune("gemm_stream_max_m", 16)
    try:
        print(f"prefill kernel M={M} K={K} N={N}", flush=True)
        qw, qz, s = make_awq(K, N, seed=M + K)
        x = make_x((M, K), seed=M)
        y = ops.w4a16_gemm(dev(x), dev(qw), dev(qz), dev(s))
        torch.cuda.synchronize()
        want = bf16_bits_to_f32(x).astype(np.float64) @ dense_f64(qw, qz, s, rounded=True)
        assert_bf16_close(bits(y), want, ulps=1.0, atol=2e-3, what="prefill kernel at small M")
    finally:
        ops.tune("gemm_stream_max_m", 0)


def test_prefill_gemm_config3(ops):
    print("gemm config3", flush=True)
    M, K, N = 2048, 4096, 14336
    qw, qz, s = make_awq(K, N, seed=3)
    x = make_x((M, K), seed=4)
    y = ops.w4a16_gemm(dev(x), dev(qw), dev(qz), dev(s))
    torch.cuda.synchronize()
    got = bits(y)
    xf = torch.from_numpy(bf16_bits_to_f32(x)).double()
    w_r = torch.from_numpy(dense_f64(qw, qz, s, rounded=True))
    want = (xf @ w_r).numpy()
    assert_bf16_close(got, want, ulps=1.0, atol=2e-3, what="config3 vs bf16-rounded-W oracle")
    # distance to the unrounded-W reference (matmul_int4_packed.cpu_reference) under the reference's gate
    w_u = torch.from_numpy(dense_f64(qw, qz, s, rounded=False))
    want_u = (xf @ w_u).numpy()
    assert oref.check_outputs(bf16_bits_to_f32(got), bf16_bits_to_f32(f32_to_bf16_bits(want_u.astype(np.float32))),
                              rtol=0.1, atol=0.05, max_mismatch_percentage=0.05, min_correlation=0.999)


def _ffn_case(ops, K, H, seed):
    print(f"ffn K={K} H={H}", flush=True)
    g = make_awq(K, H, seed=seed)
    u = make_awq(K, H, seed=seed + 1)
    d = make_awq(H, K, seed=seed + 2)
    x = make_x((K,), seed=seed + 3)
    y, h = ops.ffn_swiglu(dev(x), tuple(map(dev, g)), tuple(map(dev, u)), tuple(map(dev, d)), return_h=True)
    torch.cuda.synchronize()
    xf = bf16_bits_to_f32(x).astype(np.float64)
    g64 = xf @ dense_f64(*g)
    u64 = xf @ dense_f64(*u)
    gb = bf16_bits_to_f32(f32_to_bf16_bits(g64.astype(np.float32)))
    ub = bf16_bits_to_f32(f32_to_bf16_bits(u64.astype(np.float32)))
    h_want = oref.silu_tanh_f32(gb).astype(np.float64) * ub
    # gate/up each carry one bf16 rounding that may flip by one ulp against the float64 sum: 1 ulp on each of
    # g and u moves h by up to ~3 ulp (silu' <= 1.1)
    assert_bf16_close(bits(h), h_want, ulps=4.0, atol=2e-3, what="ffn h")
    # the down projection is checked against the oracle applied to the kernel's own h
    y_want = bf16_bits_to_f32(bits(h)).astype(np.float64) @ dense_f64(*d)
    assert_bf16_close(bits(y), y_want, ulps=1.0, atol=2e-3, what="ffn y")
    # end-to-end against the reference chain under the reference's gates
    gl1 = oawq.repack_hf_awq_linear(*g, 128)
    ul1 = oawq.repack_hf_awq_linear(*u, 128)
    dl1 = oawq.repack_hf_awq_linear(*d, 128)
    h_ref, y_ref = oref.ffn_swiglu_reference(gl1, ul1, dl1, x)
    assert oref.check_outputs(bf16_bits_to_f32(bits(h)), bf16_bits_to_f32(h_ref), rtol=0.15, atol=0.5, min_correlation=0.99)
    assert oref.check_outputs(bf16_bits_to_f32(bits(y)), bf16_bits_to_f32(y_ref), rtol=0.2, atol=2.0, min_correlation=0.99)
    mism = np.mean(bits(h) != h_ref)
    print(f"  h bit-mismatch fraction vs reference chain: {mism:.4f}", flush=True)


def test_ffn_small(ops):
    _ffn_case(ops, 256, 512, seed=20)
    _ffn_case(ops, 1024, 2048 + 128, seed=30)


def test_ffn_config4(ops):
    _ffn_case(ops, 4096, 14336, seed=40)
