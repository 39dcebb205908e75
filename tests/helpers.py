"""Shared input generators and comparison helpers for the parity tests."""
import numpy as np

from oracle import awq as oawq
from oracle.bf16 import bf16_bits_to_f32, f32_to_bf16_bits


def make_awq(K, N, gs=128, seed=0, z_range=(0, 16)):
    """Synthetic AWQ tensors in the benchmark distribution: q, z uniform uint4, scales = bf16(|N(0,1)|*0.02 + 1e-3)."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    z = rng.integers(z_range[0], z_range[1], size=(K // gs, N), dtype=np.uint8)
    s = f32_to_bf16_bits((np.abs(rng.standard_normal((K // gs, N))) * 0.02 + 1e-3).astype(np.float32))
    return oawq.pack_awq_int32(q), oawq.pack_awq_int32(z), s


def make_x(shape, seed=1):
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits(rng.standard_normal(shape).astype(np.float32))


def dense_f64(qweight, qzeros, scales, gs=128, rounded=False):
    """W[K, N] as float64: exact (q - z) * s, or the bf16-rounded weights."""
    if rounded:
        return bf16_bits_to_f32(oawq.dequant_to_bf16(qweight, qzeros, scales, gs)).astype(np.float64)
    return oawq.dequant_unrounded_f32(qweight, qzeros, scales, gs).astype(np.float64)


def bf16_ulp(v):
    """Spacing of bf16 numbers at magnitude |v| (float64 array)."""
    a = np.maximum(np.abs(np.asarray(v, dtype=np.float64)), 2.0**-126)
    return 2.0 ** (np.floor(np.log2(a)) - 7)


def assert_bf16_close(actual_bits, want_f64, ulps=1.0, atol=0.0, what=""):
    """|actual - want| <= ulps * ulp_bf16(want) + atol, elementwise."""
    got = bf16_bits_to_f32(np.asarray(actual_bits)).astype(np.float64).reshape(np.shape(want_f64))
    err = np.abs(got - want_f64)
    tol = ulps * bf16_ulp(want_f64) + atol
    bad = err > tol
    assert not bad.any(), (
        f"{what}: {int(bad.sum())}/{bad.size} elements outside {ulps} bf16 ulp + {atol}; "
        f"worst err {err.max():.4g} at {np.unravel_index(np.argmax(err - tol), err.shape)}")
