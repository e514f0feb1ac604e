"""Fused SwiGLU for MI355X, float16 storage.

Drop-in for `fused_swiglu.FastAccumFusedSwiGLU` (fused_swiglu/swiglu_f16.py:16-58).  The
reference accumulates its fp16 products in fp16 for speed on consumer GPUs; the MFMA units of
CDNA4 accumulate in fp32 at full rate, so this class is at least as accurate and the name is kept
only for compatibility."""
import torch
from torch.autograd import Function

from . import _function
from .kernels import kernels_fp16 as _kernels

_DTYPE = torch.float16


class FastAccumFusedSwiGLU(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=_DTYPE)
    def forward(ctx, input: torch.Tensor, weight_gate: torch.Tensor, weight_up: torch.Tensor) -> torch.Tensor:
        return _function.forward_training(ctx, _kernels, input, weight_gate, weight_up)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        return _function.backward(ctx, _kernels, grad_output)

    @classmethod
    def apply(cls, input, weight_gate, weight_up):
        if not _function.wants_grad(input, weight_gate, weight_up):
            return _function.forward_inference(_kernels, _DTYPE, input, weight_gate, weight_up)
        return super().apply(input, weight_gate, weight_up)
