"""bfloat16 on the host without ml_dtypes: bf16 tensors are uint16 bit patterns.

`BF16Array` tags such an array so that the runner compares it as floating point
(the reference's ml_dtypes arrays travel as int16 bits too,
python/air/backend/xrt.py:757-758).
"""

import numpy as np


class BF16Array(np.ndarray):
    """uint16 ndarray whose elements are bfloat16 bit patterns."""

    def to_f32(self):
        return to_f32(np.asarray(self))


def from_f32(a):
    """float array -> BF16Array, round-to-nearest-even."""
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    u = a.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    out = ((u.astype(np.uint64) + 0x7FFF + lsb) >> 16).astype(np.uint16)
    nan = np.isnan(a)
    if np.any(nan):
        out = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), out)
    return out.reshape(a.shape).view(BF16Array)


def from_bits(bits):
    return np.ascontiguousarray(np.asarray(bits, dtype=np.uint16)).view(BF16Array)


def to_f32(bits):
    b = np.ascontiguousarray(np.asarray(bits).view(np.uint16))
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(b.shape)


def is_bf16(a):
    if isinstance(a, BF16Array):
        return True
    return getattr(getattr(a, "dtype", None), "name", "") == "bfloat16"


def bits_of(a):
    """uint16 view of a BF16Array or an ml_dtypes bfloat16 array."""
    return np.ascontiguousarray(np.asarray(a)).view(np.uint16)
