"""`torch.library` registration of the fused SwiGLU path.

The reference offers only `FusedSwiGLU.apply` (README.md:25-38), which `torch.compile` cannot see
through.  Here the same two steps (forward launcher; gating gradient + the two gradient GEMMs) are
registered as custom operators with shape-only ("fake") implementations and an autograd formula, so
that a traced program keeps them as opaque calls into libfusedswiglu:

    fusedswiglu_amd::swiglu_forward (x, w_gate, w_up, save_preactivations) -> (out, xw_gate, xw_up)
    fusedswiglu_amd::swiglu_backward(grad_out, x, w_gate, w_up, xw_gate, xw_up,
                                     need_x, need_w_gate, need_w_up, packed) -> (dx, dw_gate, dw_up)

`swiglu(x, w_gate, w_up)` and `swiglu_packed(x, w_gate_up)` are the functional entry points.  With
`recompute=True` the forward keeps only x and the weights for the backward (fused_swiglu/swiglu.py:28
also keeps x@w_gate and x@w_up, 2*T*I elements); the backward then recomputes both products inside
the gating-gradient kernel, trading 4*T*D*I flops for that memory.  The
element type (bfloat16 or float16) is taken from the tensors; under CUDA autocast the arguments are
cast to `autocast_dtype` first, as `custom_fwd(cast_inputs=...)` does for the reference's Functions
(swiglu.py:18, swiglu_f16.py:18).  Gradient order follows swiglu.py:58: (dx, dw_gate, dw_up).
"""
from __future__ import annotations

from typing import Tuple

import torch
from torch import Tensor

from .kernels import _launch

_SUPPORTED = (torch.bfloat16, torch.float16)


def _dtype_of(x: Tensor) -> torch.dtype:
    if x.dtype not in _SUPPORTED:
        raise _launch.ShapeError(f"fused SwiGLU computes in bfloat16 or float16, got {x.dtype}")
    return x.dtype


def _empty(like: Tensor) -> Tensor:
    return like.new_empty((0,))


def _require_gpu(*tensors: Tensor) -> None:
    for t in tensors:
        if t.device.type != "cuda":
            raise _launch.ShapeError(f"fused SwiGLU needs tensors on a HIP GPU, got device '{t.device}'")


# ---- forward -----------------------------------------------------------------------------------
@torch.library.custom_op("fusedswiglu_amd::swiglu_forward", mutates_args=(), device_types="cuda")
def swiglu_forward(x: Tensor, w_gate: Tensor, w_up: Tensor,
                   save_preactivations: bool) -> Tuple[Tensor, Tensor, Tensor]:
    out, g, u = _launch.fused_swiglu_fwd(x, w_gate, w_up, _dtype_of(x),
                                         save_preactivations=save_preactivations)
    if not save_preactivations:
        g, u = _empty(out), _empty(out)
    return out, g, u


@swiglu_forward.register_fake
def _(x, w_gate, w_up, save_preactivations):
    out = x.new_empty(tuple(x.shape[:-1]) + (w_up.shape[1],))
    if save_preactivations:
        return out, torch.empty_like(out), torch.empty_like(out)
    return out, _empty(out), _empty(out)


# ---- backward ----------------------------------------------------------------------------------
@torch.library.custom_op("fusedswiglu_amd::swiglu_backward", mutates_args=(), device_types="cuda")
def swiglu_backward(grad_out: Tensor, x: Tensor, w_gate: Tensor, w_up: Tensor, xw_gate: Tensor,
                    xw_up: Tensor, need_x: bool, need_w_gate: bool, need_w_up: bool,
                    packed: bool) -> Tuple[Tensor, Tensor, Tensor]:
    """(dx, dw_gate, dw_up); a gradient that is not needed comes back with zero elements.  With
    `packed`, the second result is ONE [D, 2I] array [dw_gate | dw_up] written in place by the
    weight-gradient kernel (row stride 2I) and the third is empty: the gradient of a packed weight
    without a concatenation.  Empty xw_gate / xw_up (a forward that did not save them) switch to the
    recomputing gating-gradient kernel."""
    dtype = _dtype_of(x)
    if grad_out.dtype != dtype:
        grad_out = grad_out.to(dtype)
    if xw_gate.numel() == 0:
        d_up, d_gate = _launch.gating_grad_recompute(grad_out, x, w_gate, w_up, dtype)
    else:
        d_up, d_gate = _launch.elementwise_backward(grad_out, xw_gate, xw_up, dtype)
    dx = dw_gate = dw_up = None
    if need_x:
        dx = _launch.fused_input_grad(d_gate, d_up, w_gate, w_up, dtype)
    if need_w_gate or need_w_up:
        D, I = w_gate.shape
        if packed:
            dw_gate = torch.empty((D, 2 * I), device=x.device, dtype=dtype)
            _launch.fused_weight_grad(x, d_up, d_gate, dtype, out=(dw_gate[:, I:], dw_gate[:, :I]))
        else:
            dw_up, dw_gate = _launch.fused_weight_grad(x, d_up, d_gate, dtype)
            if not need_w_gate:
                dw_gate = None
            if not need_w_up:
                dw_up = None
    e = _empty(x)
    return (dx if dx is not None else e, dw_gate if dw_gate is not None else e.clone(),
            dw_up if dw_up is not None else e.clone())


@swiglu_backward.register_fake
def _(grad_out, x, w_gate, w_up, xw_gate, xw_up, need_x, need_w_gate, need_w_up, packed):
    D, I = w_gate.shape
    dx = torch.empty_like(x, memory_format=torch.contiguous_format) if need_x else _empty(x)
    if packed and (need_w_gate or need_w_up):
        return dx, x.new_empty((D, 2 * I)), _empty(x)
    dwg = x.new_empty((D, I)) if need_w_gate else _empty(x)
    dwu = x.new_empty((D, I)) if need_w_up else _empty(x)
    return dx, dwg, dwu


def _setup_context(ctx, inputs, output):
    x, w_gate, w_up, _ = inputs
    _, g, u = output
    ctx.save_for_backward(x, w_gate, w_up, g, u)


def _autograd_backward(ctx, grad_out, _grad_g, _grad_u):
    x, w_gate, w_up, g, u = ctx.saved_tensors
    need = ctx.needs_input_grad
    dx, dwg, dwu = swiglu_backward(grad_out.contiguous(), x, w_gate, w_up, g, u,
                                   need[0], need[1], need[2], False)
    return (dx if need[0] else None, dwg if need[1] else None, dwu if need[2] else None, None)


swiglu_forward.register_autograd(_autograd_backward, setup_context=_setup_context)


# ---- functional entry points ---------------------------------------------------------------------
def _autocast(dtype, *tensors):
    if dtype is not None and torch.is_autocast_enabled("cuda"):
        return tuple(t.to(dtype) if t.is_floating_point() else t for t in tensors)
    return tensors


def swiglu(x: Tensor, w_gate: Tensor, w_up: Tensor, autocast_dtype: torch.dtype | None = torch.bfloat16,
           recompute: bool = False) -> Tensor:
    """silu(x @ w_gate) * (x @ w_up) with weights laid out [d_model, d_intermediate]."""
    _require_gpu(x, w_gate, w_up)
    x, w_gate, w_up = _autocast(autocast_dtype, x, w_gate, w_up)
    with torch.autocast(device_type="cuda", enabled=False):
        save = torch.is_grad_enabled() and (x.requires_grad or w_gate.requires_grad or w_up.requires_grad)
        return swiglu_forward(x, w_gate, w_up, save and not recompute)[0]


class _PackedSwiGLU(torch.autograd.Function):
    """One [D, 2I] weight holding gate columns then up columns.  The kernels take the two halves as
    strided views (row stride 2I), and the weight gradient is written straight into one [D, 2I]
    array, so packing costs no copies in either direction."""

    @staticmethod
    def forward(ctx, x, w_gate_up, recompute):
        I = w_gate_up.shape[1] // 2
        w_gate, w_up = w_gate_up[:, :I], w_gate_up[:, I:]
        out, g, u = swiglu_forward(x, w_gate, w_up, not recompute)
        ctx.save_for_backward(x, w_gate_up, g, u)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w_gate_up, g, u = ctx.saved_tensors
        I = w_gate_up.shape[1] // 2
        need_x, need_w = ctx.needs_input_grad[:2]
        dx, dw, _ = swiglu_backward(grad_out.contiguous(), x, w_gate_up[:, :I], w_gate_up[:, I:], g, u,
                                    need_x, need_w, need_w, True)
        return (dx if need_x else None), (dw if need_w else None), None


def swiglu_packed(x: Tensor, w_gate_up: Tensor, autocast_dtype: torch.dtype | None = torch.bfloat16,
                  recompute: bool = False) -> Tensor:
    """SwiGLU with a packed weight [d_model, 2*d_intermediate] = [w_gate | w_up]."""
    if w_gate_up.ndim != 2 or w_gate_up.shape[1] % 2:
        raise _launch.ShapeError("packed weight must be [d_model, 2*d_intermediate]")
    _require_gpu(x, w_gate_up)
    x, w_gate_up = _autocast(autocast_dtype, x, w_gate_up)
    with torch.autocast(device_type="cuda", enabled=False):
        if torch.is_grad_enabled() and (x.requires_grad or w_gate_up.requires_grad):
            return _PackedSwiGLU.apply(x, w_gate_up, recompute)
        I = w_gate_up.shape[1] // 2
        return swiglu_forward(x, w_gate_up[:, :I], w_gate_up[:, I:], False)[0]
