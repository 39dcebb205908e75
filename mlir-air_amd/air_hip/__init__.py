"""air_hip - MI355X (gfx950) host side of the AWQ int4 / W4A16 path.

The package mirrors the reference's example/runner interface
(programming_examples/*/int4_awq/*.py, python/air/backend/xrt_runner.py) on top
of the C ABI in include/w4a16.h.  There is no CPU fallback: every op raises if
the HIP library is not built.
"""

from . import awq, bf16  # noqa: F401
from ._lib import LibraryNotBuiltError, W4A16Error, library_path, load_library  # noqa: F401

__all__ = ["awq", "bf16", "load_library", "library_path", "LibraryNotBuiltError", "W4A16Error"]
