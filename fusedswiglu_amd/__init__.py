"""MI355X-native fused SwiGLU forward/backward (hand-written gfx950 HIP kernels behind a C ABI).

Exports the same two names as the reference package (fused_swiglu/__init__.py:1-2)."""
from .swiglu import FusedSwiGLU
from .swiglu_f16 import FastAccumFusedSwiGLU

__all__ = ["FusedSwiGLU", "FastAccumFusedSwiGLU"]
