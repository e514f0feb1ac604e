"""MI355X-native fused SwiGLU forward/backward (hand-written gfx950 HIP kernels behind a C ABI).

Exports the same two names as the reference package (fused_swiglu/__init__.py:1-2), plus the
`torch.library` operators (`swiglu`, `swiglu_packed`) and the `SwiGLU` module built on them."""
from .swiglu import FusedSwiGLU
from .swiglu_f16 import FastAccumFusedSwiGLU
from .ops import swiglu, swiglu_packed
from .module import SwiGLU

__all__ = ["FusedSwiGLU", "FastAccumFusedSwiGLU", "swiglu", "swiglu_packed", "SwiGLU"]
