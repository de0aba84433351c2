"""axiom_amd — MI355X (gfx950) GEMM backend for Axiom.

The product is two shared libraries under axiom_amd/lib/ (built by axiom_amd/csrc/Makefile):
libaxhip.so (HIP kernels behind the C ABI of include/axhip.h) and libaxiom_hip.so (the C
host core and the ``ax_hip_ops`` backend vtable).  The Python modules here are thin ctypes
loaders used by the tests and the benchmark; there is no CPU fallback.
"""
from .hip import AxHip, AxHipError, DeviceArray  # noqa: F401

__all__ = ["AxHip", "AxHipError", "DeviceArray"]
