"""TEST INFRASTRUCTURE ONLY.

CPU restatement (NumPy + a small C file) of the reference's AWQ int4 / W4A16
algorithms.  Only tests, the smoke check and the benchmark's CPU-baseline leg
may import this package; the product path never does and has no CPU fallback.
"""

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libw4a16_oracle.so")


def build_c_oracle():
    """Compile oracle/w4a16_oracle.c with gcc (idempotent)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "-B"])
    return _SO


def load_c_oracle():
    """ctypes handle to the C restatement; builds it when missing."""
    if not os.path.exists(_SO):
        build_c_oracle()
    lib = ctypes.CDLL(_SO)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.oracle_matvec_loop.argtypes = [vp, vp, vp, vp, ci, ci, ci, vp]
    lib.oracle_matvec_loop.restype = None
    lib.oracle_dequant_awq.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    lib.oracle_dequant_awq.restype = None
    return lib
