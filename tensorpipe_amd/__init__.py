"""MI355X-native device-channel layer with TensorPipe's channel plugin surface.

The compute path lives in csrc/ (HIP kernels behind the C ABI in include/);
this package is the thin Python face used by tests and the bench.
"""
from . import _native  # noqa: F401

__all__ = ["_native"]
