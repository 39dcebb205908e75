"""GPU parity on weights QUANTISED FROM A bf16 MATRIX (fake_quantize_awq_int4, awq_pack.py:287-316) instead of uniform
random nibbles: zero points cluster and hit both ends, scales spread over decades, constant and one-sided groups occur.
Dequant bit-exact; GEMV, the batched kernel and the tiled kernel within one bf16 ulp of the float64 product plus the
fp32 accumulation slack 2^-16 * sum |x w|; and the switch of w4a16_gemm_stream_bf16 from exact to bf16-rounded
weights between M = 128 and M = 129."""
import numpy as np
import pytest
import torch

from helpers import bf16_ulp, dense_f64, make_awq, make_x
from oracle import awq as oawq, reference as oref
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(a).cuda()


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _quantised(N, K, seed):
    """A weight [N, K] with per-row magnitudes over three decades, outliers, a constant group and a one-sided group,
    quantised by the host quantiser; returns the AutoAWQ tensors and the original float32 matrix."""
    from air_hip import awq, bf16
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.02 * 10.0 ** rng.uniform(-2, 1, (N, 1))).astype(np.float32)
    w[rng.integers(0, N, 64), rng.integers(0, K, 64)] *= 25.0     # outliers stretch their group's range
    w[1, :128] = 0.0625                                           # constant group
    w[2, 128:256] = np.abs(w[2, 128:256]) + 0.01                  # one-sided group: zero point clips to 0
    w[3, 128:256] = -np.abs(w[3, 128:256]) - 0.01                 # ... and to 15
    wb = bf16.from_f32(w)
    a_q, a_s, a_z = awq.fake_quantize_awq_int4(wb, 128)
    qw, qz, s = awq.awq_from_l1(a_q, a_s, a_z)
    return qw, qz, bf16.bits_of(s), bf16.to_f32(bf16.bits_of(wb))


def _close(got_bits, want, slack, what):
    got = bf16_bits_to_f32(got_bits).astype(np.float64).reshape(want.shape)
    tol = bf16_ulp(want) + slack
    bad = np.abs(got - want) > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside 1 ulp + slack, worst {np.abs(got - want).max()}"


def test_products_on_weights_quantised_from_bf16():
    from air_hip import ops
    K, N = 2048, 1024
    qw, qz, s, w_orig = _quantised(N, K, seed=3)
    z = oawq.unpack_awq_int32(qz)
    assert z.min() == 0 and z.max() == 15 and np.bincount(z.reshape(-1), minlength=16)[8] > 5 * np.bincount(z.reshape(-1), minlength=16)[1]
    sf = bf16_bits_to_f32(s)
    assert sf.max() / sf[sf > 1e-6].min() > 300           # scales over decades
    print("quantised weights: dequant", flush=True)
    tri = (dev(qw), dev(qz), dev(s))
    assert np.array_equal(bits(ops.awq_dequant(*tri)), oawq.dequant_to_bf16(qw, qz, s, 128))
    sw = ops.repack_stream(*tri)
    W = dense_f64(qw, qz, s)
    Wr = dense_f64(qw, qz, s, rounded=True)
    for M in (1, 16, 64, 300):
        print(f"quantised weights: M={M}", flush=True)
        x = make_x((M, K), seed=10 + M)
        xf = bf16_bits_to_f32(x).astype(np.float64)
        y = ops.w4a16_gemm_stream(dev(x), sw) if M > 1 else ops.w4a16_gemv_stream(dev(x[0]), sw).reshape(1, N)
        torch.cuda.synchronize()
        Wm = Wr if M > 128 else W
        _close(bits(y), xf @ Wm, 2.0**-16 * (np.abs(xf) @ np.abs(Wm)), f"M={M}")
        # and the quantised product tracks the product with the matrix it was quantised from
        ref = xf @ w_orig.T.astype(np.float64)
        assert np.corrcoef(bf16_bits_to_f32(bits(y)).reshape(-1), ref.reshape(-1))[0, 1] > 0.99
    # checkpoint-layout kernel on the same tensors
    x = make_x((K,), seed=77)
    y = ops.w4a16_gemv(dev(x), *tri)
    torch.cuda.synchronize()
    xf = bf16_bits_to_f32(x).astype(np.float64)
    _close(bits(y), xf @ W, 2.0**-16 * (np.abs(xf) @ np.abs(W)), "checkpoint-layout gemv")


def test_gemm_stream_switches_to_rounded_weights_above_128_rows():
    """w4a16_gemm_stream_bf16 multiplies the exact weights (q - z) s up to M = 128 (batched whole-K kernel) and the
    bf16-rounded weights of the dense dequant from M = 129 on (tiled kernel); the reference's cpu_reference multiplies
    unrounded weights at every M (matmul_int4_packed.py:89-105).  Each side is within one ulp of its own float64
    product, both pass the reference's gate against the unrounded product, and rows 0..127 of the two agree to the
    weight rounding (2^-9 relative per weight)."""
    from air_hip import ops
    K, N = 1024, 512
    qw, qz, s = make_awq(K, N, seed=41)
    sw = ops.repack_stream(dev(qw), dev(qz), dev(s))
    x = make_x((129, K), seed=42)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    W, Wr = dense_f64(qw, qz, s), dense_f64(qw, qz, s, rounded=True)
    print("gemm stream M=128", flush=True)
    y128 = bits(ops.w4a16_gemm_stream(dev(x[:128]), sw))
    print("gemm stream M=129", flush=True)
    y129 = bits(ops.w4a16_gemm_stream(dev(x), sw))
    _close(y128, xf[:128] @ W, 2e-3, "M=128 against exact weights")
    _close(y129, xf @ Wr, 2e-3, "M=129 against rounded weights")
    unrounded = bf16_bits_to_f32(f32_to_bf16_bits((xf @ W).astype(np.float32)))
    for got, rows in ((y128, 128), (y129, 129)):
        assert oref.check_outputs(bf16_bits_to_f32(got), unrounded[:rows], rtol=0.1, atol=0.05, max_mismatch_percentage=0.05,
                                  min_correlation=0.999)
    a, b = bf16_bits_to_f32(y128).astype(np.float64), bf16_bits_to_f32(y129[:128]).astype(np.float64)
    assert np.any(y128 != y129[:128])                       # they are different sums
    assert np.all(np.abs(a - b) <= 2 * bf16_ulp(a) + 2.0**-9 * (np.abs(xf[:128]) @ np.abs(W)))   # |sum x (W - bf16 W)| <= 2^-9 sum |x W|
