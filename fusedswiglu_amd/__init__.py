"""MI355X-native fused SwiGLU forward/backward (hand-written gfx950 HIP kernels behind a C ABI).

Exports the same two names as the reference package (fused_swiglu/__init__.py:1-2), plus the
`torch.library` operators (`swiglu`, `swiglu_packed`, `down_proj`, `swiglu_mlp`) and the `SwiGLU` /
`SwiGLUMLP` modules built on them."""
from .swiglu import FusedSwiGLU
from .swiglu_f16 import FastAccumFusedSwiGLU
from .ops import down_proj, swiglu, swiglu_mlp, swiglu_packed
from .module import SwiGLU, SwiGLUMLP

__all__ = ["FusedSwiGLU", "FastAccumFusedSwiGLU", "swiglu", "swiglu_packed", "down_proj", "swiglu_mlp",
           "SwiGLU", "SwiGLUMLP"]
