"""TEST INFRASTRUCTURE ONLY - bfloat16 helpers for the CPU oracle.

NumPy has no bfloat16 dtype and the reference's `ml_dtypes` is not installed,
so bf16 tensors are carried as uint16 bit patterns.  Only `tests/`, the smoke
check and the CPU-baseline leg of the benchmark may import this package; the
product never does.

The reference rounds with `ndarray.astype(ml_dtypes.bfloat16)`
(e.g. programming_examples/llms/llama32_1b_int4/awq_repacker.py:82), which is
round-to-nearest-even from float32.  float64 inputs are first rounded to
float32 and then to bf16 (ml_dtypes casts go through float).

Pinned by tests/test_oracle_bf16.py against `torch.Tensor.to(torch.bfloat16)`
and hand-computed tie cases.
"""

import numpy as np


def f32_to_bf16_bits(a):
    """float array -> uint16 bf16 bit patterns, round-to-nearest-even."""
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    u = a.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u.astype(np.uint64) + 0x7FFF + lsb) >> 16).astype(np.uint16)
    # NaN: keep sign and exponent, force a quiet mantissa bit.
    nan = np.isnan(a)
    if np.any(nan):
        rounded = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), rounded)
    return rounded.reshape(a.shape)


def bf16_bits_to_f32(bits):
    """uint16 bf16 bit patterns -> float32 values (exact)."""
    b = np.ascontiguousarray(np.asarray(bits, dtype=np.uint16))
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(b.shape)


def round_to_bf16(a):
    """Values rounded to bf16, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a))
