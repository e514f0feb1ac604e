"""Shared body of the two autograd Functions (bf16 and fp16 differ only in the launcher module
and the autocast dtype, exactly as fused_swiglu/swiglu.py and swiglu_f16.py do)."""
from __future__ import annotations

import torch


def autocast_inputs(dtype: torch.dtype, *tensors: torch.Tensor):
    """What torch.amp.custom_fwd(cast_inputs=dtype) does to tensor arguments: under CUDA autocast,
    floating-point GPU tensors are cast to `dtype`; outside autocast nothing is touched."""
    if torch.is_autocast_enabled("cuda"):
        return tuple(t.to(dtype) if (t.is_floating_point() and t.is_cuda) else t for t in tensors)
    return tensors


def wants_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def forward_inference(kernels, dtype, input, weight_gate, weight_up):
    """Forward without an autograd node: the pre-activations are neither stored nor allocated."""
    input, weight_gate, weight_up = autocast_inputs(dtype, input, weight_gate, weight_up)
    with torch.autocast(device_type="cuda", enabled=False):
        out, _, _ = kernels.fused_swiglu_fwd(input, weight_gate, weight_up, save_preactivations=False)
    return out


def forward_training(ctx, kernels, input, weight_gate, weight_up):
    """fused_swiglu/swiglu.py:19-30: launch, save (x, Wg, Wu, x@Wg, x@Wu), return out."""
    out, xw_gate, xw_up = kernels.fused_swiglu_fwd(input, weight_gate, weight_up)
    ctx.save_for_backward(input, weight_gate, weight_up, xw_gate, xw_up)
    return out


def backward(ctx, kernels, grad_output):
    """fused_swiglu/swiglu.py:34-58.  Returns (grad_input, grad_weight_gate, grad_weight_up).
    One library call, three launches: gating gradient, input-gradient dual GEMM, weight-gradient dual GEMM
    (reduced over all tokens, so the reference's per-batch partials and `unbroadcast` sum disappear).
    Gradients nobody asked for (ctx.needs_input_grad) are skipped."""
    input, weight_gate, weight_up, xw_gate, xw_up = ctx.saved_tensors
    if grad_output.dtype != xw_gate.dtype:
        grad_output = grad_output.to(xw_gate.dtype)
    need = ctx.needs_input_grad
    grad_input, grad_weight_gate, grad_weight_up = kernels.swiglu_backward(
        grad_output, input, weight_gate, weight_up, xw_gate, xw_up,
        need_input_grad=need[0], need_weight_grad=need[1] or need[2])
    return grad_input, grad_weight_gate if need[1] else None, grad_weight_up if need[2] else None
