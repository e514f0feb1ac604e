"""Fused SwiGLU for MI355X, bfloat16 storage, fp32 MFMA accumulation.

Drop-in for `fused_swiglu.FusedSwiGLU` (fused_swiglu/swiglu.py:16-58): same call,
`FusedSwiGLU.apply(input, weight_gate, weight_up)` with weights laid out [d_model, d_intermediate],
same autocast behaviour (inputs are cast to bfloat16 only under torch.autocast), same gradients
(grad_input, grad_weight_gate, grad_weight_up)."""
import torch
from torch.autograd import Function

from . import _function
from .kernels import kernels_bf16 as _kernels

_DTYPE = torch.bfloat16


class FusedSwiGLU(Function):
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
        # no gradient can flow: skip the autograd node and the two pre-activation stores
        if not _function.wants_grad(input, weight_gate, weight_up):
            return _function.forward_inference(_kernels, _DTYPE, input, weight_gate, weight_up)
        return super().apply(input, weight_gate, weight_up)
