"""`torch.library` registration of the fused SwiGLU path.

The reference offers only `FusedSwiGLU.apply` (README.md:25-38), which `torch.compile` cannot see
through.  Here the same two steps (forward launcher; gating gradient + the two gradient GEMMs) are
registered as custom operators with shape-only ("fake") implementations and an autograd formula, so
that a traced program keeps them as opaque calls into libfusedswiglu:

    fusedswiglu_amd::swiglu_forward (x, w_gate, w_up, save_preactivations, weights_out_in) -> (out, xw_gate, xw_up)
    fusedswiglu_amd::swiglu_backward(grad_out, x, w_gate, w_up, xw_gate, xw_up,
                                     need_x, need_w_gate, need_w_up, packed, weights_out_in) -> (dx, dw_gate, dw_up)
    fusedswiglu_amd::down_proj_forward (act, w_down, weights_out_in) -> y
    fusedswiglu_amd::down_proj_backward(grad_y, act, w_down, need_act, need_w, weights_out_in) -> (d_act, d_w_down)

`swiglu(x, w_gate, w_up)`, `swiglu_packed(x, w_gate_up)`, `down_proj(act, w_down)` and `swiglu_mlp(x, w_gate,
w_up, w_down)` are the functional entry points.  `weights_out_in=True` means the weights are stored like
`nn.Linear.weight` (w_gate, w_up [d_intermediate, d_model]; w_down [d_model, d_intermediate]) and are read in
place; the default is the reference's layout (w_gate, w_up [d_model, d_intermediate], README.md:26-27; w_down
[d_intermediate, d_model]).  With
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
def swiglu_forward(x: Tensor, w_gate: Tensor, w_up: Tensor, save_preactivations: bool,
                   weights_out_in: bool = False) -> Tuple[Tensor, Tensor, Tensor]:
    out, g, u = _launch.fused_swiglu_fwd(x, w_gate, w_up, _dtype_of(x),
                                         save_preactivations=save_preactivations, weights_out_in=weights_out_in)
    if not save_preactivations:
        g, u = _empty(out), _empty(out)
    return out, g, u


@swiglu_forward.register_fake
def _(x, w_gate, w_up, save_preactivations, weights_out_in=False):
    out = x.new_empty(tuple(x.shape[:-1]) + (w_up.shape[0 if weights_out_in else 1],))
    if save_preactivations:
        return out, torch.empty_like(out), torch.empty_like(out)
    return out, _empty(out), _empty(out)


# ---- backward ----------------------------------------------------------------------------------
@torch.library.custom_op("fusedswiglu_amd::swiglu_backward", mutates_args=(), device_types="cuda")
def swiglu_backward(grad_out: Tensor, x: Tensor, w_gate: Tensor, w_up: Tensor, xw_gate: Tensor,
                    xw_up: Tensor, need_x: bool, need_w_gate: bool, need_w_up: bool,
                    packed: bool, weights_out_in: bool = False) -> Tuple[Tensor, Tensor, Tensor]:
    """(dx, dw_gate, dw_up); a gradient that is not needed comes back with zero elements.  With
    `packed`, the second result is ONE array [dw_gate | dw_up] ([D, 2I]; [2I, D] with weights_out_in)
    written in place by the weight-gradient kernel and the third is empty: the gradient of a packed
    weight without a concatenation.  Empty xw_gate / xw_up (a forward that did not save them) switch to
    the recomputing gating-gradient kernel."""
    dtype = _dtype_of(x)
    oi = weights_out_in
    if grad_out.dtype != dtype:
        grad_out = grad_out.to(dtype)
    e = _empty(x)
    if xw_gate.numel() != 0 and not packed:
        # the common case in one library call (gating gradient, weight gradient, input gradient)
        dx, dw_gate, dw_up = _launch.swiglu_backward(grad_out, x, w_gate, w_up, xw_gate, xw_up, dtype, need_input_grad=need_x,
                                                     need_weight_grad=need_w_gate or need_w_up, weights_out_in=oi)
        return (dx if dx is not None else e, dw_gate if need_w_gate else e.clone(), dw_up if need_w_up else e.clone())
    if xw_gate.numel() == 0:
        d_up, d_gate = _launch.gating_grad_recompute(grad_out, x, w_gate, w_up, dtype, weights_out_in=oi)
    else:
        d_up, d_gate = _launch.elementwise_backward(grad_out, xw_gate, xw_up, dtype)
    dx = dw_gate = dw_up = None
    # the weight gradient first: the input gradient then finds d_gate and d_up in the memory-side cache
    if need_w_gate or need_w_up:
        if packed and oi:
            I, D = w_gate.shape
            dw_gate = torch.empty((2 * I, D), device=x.device, dtype=dtype)
            _launch.fused_weight_grad(x, d_up, d_gate, dtype, out=(dw_gate[I:], dw_gate[:I]), weights_out_in=True)
        elif packed:
            D, I = w_gate.shape
            dw_gate = torch.empty((D, 2 * I), device=x.device, dtype=dtype)
            _launch.fused_weight_grad(x, d_up, d_gate, dtype, out=(dw_gate[:, I:], dw_gate[:, :I]))
        else:
            dw_up, dw_gate = _launch.fused_weight_grad(x, d_up, d_gate, dtype, weights_out_in=oi)
            if not need_w_gate:
                dw_gate = None
            if not need_w_up:
                dw_up = None
    if need_x:
        dx = _launch.fused_input_grad(d_gate, d_up, w_gate, w_up, dtype, weights_out_in=oi)
    return (dx if dx is not None else e, dw_gate if dw_gate is not None else e.clone(),
            dw_up if dw_up is not None else e.clone())


@swiglu_backward.register_fake
def _(grad_out, x, w_gate, w_up, xw_gate, xw_up, need_x, need_w_gate, need_w_up, packed, weights_out_in=False):
    r, c = w_gate.shape
    dx = torch.empty_like(x, memory_format=torch.contiguous_format) if need_x else _empty(x)
    if packed and (need_w_gate or need_w_up):
        return dx, x.new_empty((2 * r, c) if weights_out_in else (r, 2 * c)), _empty(x)
    dwg = x.new_empty((r, c)) if need_w_gate else _empty(x)
    dwu = x.new_empty((r, c)) if need_w_up else _empty(x)
    return dx, dwg, dwu


def _setup_context(ctx, inputs, output):
    x, w_gate, w_up, _, weights_out_in = inputs
    _, g, u = output
    ctx.save_for_backward(x, w_gate, w_up, g, u)
    ctx.weights_out_in = weights_out_in


def _autograd_backward(ctx, grad_out, _grad_g, _grad_u):
    x, w_gate, w_up, g, u = ctx.saved_tensors
    need = ctx.needs_input_grad
    dx, dwg, dwu = swiglu_backward(grad_out.contiguous(), x, w_gate, w_up, g, u,
                                   need[0], need[1], need[2], False, ctx.weights_out_in)
    return (dx if need[0] else None, dwg if need[1] else None, dwu if need[2] else None, None, None)


swiglu_forward.register_autograd(_autograd_backward, setup_context=_setup_context)


# ---- the down projection that follows --------------------------------------------------------------
@torch.library.custom_op("fusedswiglu_amd::down_proj_forward", mutates_args=(), device_types="cuda")
def down_proj_forward(act: Tensor, w_down: Tensor, weights_out_in: bool = False) -> Tensor:
    return _launch.down_proj_forward(act, w_down, _dtype_of(act), weights_out_in=weights_out_in)


@down_proj_forward.register_fake
def _(act, w_down, weights_out_in=False):
    return act.new_empty(tuple(act.shape[:-1]) + (w_down.shape[0 if weights_out_in else 1],))


@torch.library.custom_op("fusedswiglu_amd::down_proj_backward", mutates_args=(), device_types="cuda")
def down_proj_backward(grad_y: Tensor, act: Tensor, w_down: Tensor, need_act: bool, need_w: bool,
                       weights_out_in: bool = False) -> Tuple[Tensor, Tensor]:
    """(grad_act, grad_w_down); a gradient that is not needed comes back with zero elements."""
    dtype = _dtype_of(act)
    if grad_y.dtype != dtype:
        grad_y = grad_y.to(dtype)
    e = _empty(act)
    d_act = _launch.down_proj_input_grad(grad_y, w_down, dtype, weights_out_in=weights_out_in) if need_act else e
    d_w = _launch.down_proj_weight_grad(act, grad_y, dtype, weights_out_in=weights_out_in) if need_w else e.clone()
    return d_act, d_w


@down_proj_backward.register_fake
def _(grad_y, act, w_down, need_act, need_w, weights_out_in=False):
    d_act = torch.empty_like(act, memory_format=torch.contiguous_format) if need_act else _empty(act)
    return d_act, (act.new_empty(tuple(w_down.shape)) if need_w else _empty(act))


def _down_setup(ctx, inputs, output):
    act, w_down, weights_out_in = inputs
    ctx.save_for_backward(act, w_down)
    ctx.weights_out_in = weights_out_in


def _down_backward(ctx, grad_y):
    act, w_down = ctx.saved_tensors
    need = ctx.needs_input_grad
    d_act, d_w = down_proj_backward(grad_y.contiguous(), act, w_down, need[0], need[1], ctx.weights_out_in)
    return (d_act if need[0] else None, d_w if need[1] else None, None)


down_proj_forward.register_autograd(_down_backward, setup_context=_down_setup)


# ---- functional entry points ---------------------------------------------------------------------
def _autocast(dtype, *tensors):
    if dtype is not None and torch.is_autocast_enabled("cuda"):
        return tuple(t.to(dtype) if t.is_floating_point() else t for t in tensors)
    return tensors


def swiglu(x: Tensor, w_gate: Tensor, w_up: Tensor, autocast_dtype: torch.dtype | None = torch.bfloat16,
           recompute: bool = False, weights_out_in: bool = False) -> Tensor:
    """silu(x @ w_gate) * (x @ w_up) with weights laid out [d_model, d_intermediate], or
    silu(x @ w_gate.T) * (x @ w_up.T) with nn.Linear-style [d_intermediate, d_model] weights
    (`weights_out_in=True`), which are read in place."""
    _require_gpu(x, w_gate, w_up)
    x, w_gate, w_up = _autocast(autocast_dtype, x, w_gate, w_up)
    with torch.autocast(device_type="cuda", enabled=False):
        save = torch.is_grad_enabled() and (x.requires_grad or w_gate.requires_grad or w_up.requires_grad)
        return swiglu_forward(x, w_gate, w_up, save and not recompute, weights_out_in)[0]


def down_proj(act: Tensor, w_down: Tensor, autocast_dtype: torch.dtype | None = torch.bfloat16,
              weights_out_in: bool = False) -> Tensor:
    """act @ w_down with w_down [d_intermediate, d_model] (act @ w_down.T for nn.Linear-style
    [d_model, d_intermediate] with `weights_out_in=True`)."""
    _require_gpu(act, w_down)
    act, w_down = _autocast(autocast_dtype, act, w_down)
    with torch.autocast(device_type="cuda", enabled=False):
        return down_proj_forward(act, w_down, weights_out_in)


def swiglu_mlp(x: Tensor, w_gate: Tensor, w_up: Tensor, w_down: Tensor,
               autocast_dtype: torch.dtype | None = torch.bfloat16, recompute: bool = False,
               weights_out_in: bool = False) -> Tensor:
    """The whole gated MLP block: (silu(x Wg) * (x Wu)) W_down, chaining the fused SwiGLU and the down
    projection (which the reference leaves to its caller, README.md:25-38)."""
    return down_proj(swiglu(x, w_gate, w_up, autocast_dtype, recompute, weights_out_in), w_down,
                     autocast_dtype, weights_out_in)


def _halves(w_gate_up: Tensor, weights_out_in: bool):
    """(w_gate, w_up) views of a packed weight: column halves of [D, 2I], row halves of [2I, D]."""
    if weights_out_in:
        I = w_gate_up.shape[0] // 2
        return w_gate_up[:I], w_gate_up[I:]
    I = w_gate_up.shape[1] // 2
    return w_gate_up[:, :I], w_gate_up[:, I:]


class _PackedSwiGLU(torch.autograd.Function):
    """One weight holding gate then up: [D, 2I] (gate columns, up columns) or, nn.Linear style, [2I, D]
    (gate rows, up rows).  The kernels take the two halves as views, and the weight gradient is written
    straight into one array of the same shape, so packing costs no copies in either direction."""

    @staticmethod
    def forward(ctx, x, w_gate_up, recompute, weights_out_in):
        w_gate, w_up = _halves(w_gate_up, weights_out_in)
        out, g, u = swiglu_forward(x, w_gate, w_up, not recompute, weights_out_in)
        ctx.save_for_backward(x, w_gate_up, g, u)
        ctx.weights_out_in = weights_out_in
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w_gate_up, g, u = ctx.saved_tensors
        w_gate, w_up = _halves(w_gate_up, ctx.weights_out_in)
        need_x, need_w = ctx.needs_input_grad[:2]
        dx, dw, _ = swiglu_backward(grad_out.contiguous(), x, w_gate, w_up, g, u,
                                    need_x, need_w, need_w, True, ctx.weights_out_in)
        return (dx if need_x else None), (dw if need_w else None), None, None


def swiglu_packed(x: Tensor, w_gate_up: Tensor, autocast_dtype: torch.dtype | None = torch.bfloat16,
                  recompute: bool = False, weights_out_in: bool = False) -> Tensor:
    """SwiGLU with a packed weight [d_model, 2*d_intermediate] = [w_gate | w_up] (or, with
    `weights_out_in`, [2*d_intermediate, d_model] = gate rows then up rows)."""
    if w_gate_up.ndim != 2 or w_gate_up.shape[0 if weights_out_in else 1] % 2:
        raise _launch.ShapeError("packed weight must be [d_model, 2*d_intermediate] (or [2*d_intermediate, d_model])")
    _require_gpu(x, w_gate_up)
    x, w_gate_up = _autocast(autocast_dtype, x, w_gate_up)
    with torch.autocast(device_type="cuda", enabled=False):
        if torch.is_grad_enabled() and (x.requires_grad or w_gate_up.requires_grad):
            return _PackedSwiGLU.apply(x, w_gate_up, recompute, weights_out_in)
        w_gate, w_up = _halves(w_gate_up, weights_out_in)
        return swiglu_forward(x, w_gate, w_up, False, weights_out_in)[0]
