"""Backend boundary of the W4A16 path: the HIP counterpart of air.backend
(python/air/backend/abc.py, xrt.py, xrt_runner.py in the reference)."""

from .abc import AirBackend, AirBackendError  # noqa: F401
from .hip import HIPBackend, HipModule  # noqa: F401
from .hip_runner import HIPRunner  # noqa: F401
