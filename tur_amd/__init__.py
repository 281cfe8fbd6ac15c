"""tur_amd — MI355X-native GGUF quantized linear layers (Q8_0, Q4_K, Q5_K, Q6_K).

The product is ``libturq.so`` (HIP kernels + C ABI, see ``include/turq.h``).  This package is the
thin Python host side used by tests, the benchmark and Python callers: ``tur_amd.capi`` binds the
C ABI with ctypes, ``tur_amd.qlinear`` mirrors the reference's ``QVarBuilder`` / ``QMatMul`` /
``LinearX`` interface on top of it.  Nothing here computes on the CPU: without the built library
(or without a GPU) the calls fail loudly.
"""
from . import synth  # noqa: F401

__all__ = ["synth", "capi", "qlinear", "gguf"]
