"""sarek-hip: MI355X (gfx950) backend for the Sarek/SPOC hot path.

The product is the C-ABI library ``libsarek_hip.so`` (see ``include/sarek_hip.h``).
This package is the thin Python front end used by the tests and the benchmark:
it loads the library with ctypes and passes device pointers of torch tensors.
There is no CPU fallback: importing :mod:`spoc_amd.hip` raises if the library is
not built.
"""
from . import hip  # noqa: F401

__all__ = ["hip"]
