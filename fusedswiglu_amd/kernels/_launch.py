"""dtype-generic host launchers: torch tensors in, raw device pointers through the C ABI.

PyTorch is plumbing here (device memory, the current HIP stream); all arithmetic happens in
libfusedswiglu.  Mirrors the launcher seam of the reference
(fused_swiglu/kernels/kernels_bf16.py:162-206, :236-255, :385-412) with these differences:
  * x may have any number (>= 1) of leading dimensions; they are flattened into T tokens
    (the reference insists on exactly 3-D input, kernels_bf16.py:178-180);
  * weight gradients come back already reduced over all tokens, shape [D, I];
  * the input gradient has its own launcher instead of two torch matmuls (swiglu.py:45);
  * `weights_out_in=True` takes the weights (and returns their gradients) in nn.Linear's [I, D]
    layout instead of the reference's [D, I] (README.md:26-27), without transposing anything;
  * down_proj_forward / _input_grad / _weight_grad are the down projection that follows the SwiGLU
    in an MLP block (the reference leaves it to the caller, README.md:25-38).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _abi


class ShapeError(AssertionError, ValueError):
    """Bad shape / dtype / device.  The reference signals these with `assert`
    (kernels_bf16.py:170-182); this is an AssertionError and a ValueError at once."""


_DTYPE_CODE = {torch.bfloat16: _abi.DTYPE_BF16, torch.float16: _abi.DTYPE_FP16}


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ShapeError(msg)


def _check_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise ShapeError(f"fused SwiGLU needs tensors on a HIP GPU, got device '{dev}'")
    for t in tensors[1:]:
        if t.device != dev:
            raise ShapeError(f"all tensors must be on the same device ({t.device} vs {dev})")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(dev: torch.device) -> int:
    """Handle of torch's current HIP stream on `dev` (without building a Stream object when torch offers
    the raw getter: this runs four times per training step)."""
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


class _on_device:
    """`with torch.cuda.device(dev)` that costs nothing when `dev` is already the current device (the usual
    case); kernels are launched on the current device, so the guard is needed only when it differs."""
    __slots__ = ("guard",)

    def __init__(self, dev: torch.device):
        self.guard = None if dev.index is None or torch.cuda.current_device() == dev.index else torch.cuda.device(dev)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


def _rows(t: torch.Tensor) -> torch.Tensor:
    """2-D [rows, cols] view with unit inner stride (copies only if it must)."""
    if t.ndim == 2 and t.stride(1) == 1 and (t.shape[0] <= 1 or t.stride(0) >= t.shape[1]):
        return t
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(-1) != 1 or (t2.shape[0] > 1 and t2.stride(0) < t2.shape[1]):
        t2 = t2.contiguous()
    return t2


def _workspace(step: int, T: int, D: int, I: int, dev: torch.device):
    """(tensor or None, bytes) of fp32 scratch that lets a small gradient GEMM split its reduction
    over several workgroups; the library says how much it wants (0 for problems that fill the chip)."""
    nbytes = int(_abi.lib().fsw_workspace_bytes(step, T, D, I))
    if nbytes <= 0:
        return None, 0
    return torch.empty(nbytes, device=dev, dtype=torch.uint8), nbytes


def _ld(t2: torch.Tensor) -> int:
    return t2.stride(0) if t2.shape[0] > 1 else t2.shape[1]


def _code(dtype: torch.dtype, weights_out_in: bool) -> int:
    return _DTYPE_CODE[dtype] | (_abi.WEIGHTS_OUT_IN if weights_out_in else 0)


def _weight_dims(w: torch.Tensor, weights_out_in: bool) -> Tuple[int, int]:
    """(D, I) of a gate/up weight in either layout."""
    return (w.shape[1], w.shape[0]) if weights_out_in else (w.shape[0], w.shape[1])


def fused_swiglu_fwd(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, dtype: torch.dtype,
                     save_preactivations: bool = True, weights_out_in: bool = False
                     ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """out = silu(x @ w_gate) * (x @ w_up); returns (out, x@w_gate, x@w_up) like
    kernels_bf16.py:162-206.  With save_preactivations=False the two pre-activation arrays are
    neither allocated nor written and None is returned for them."""
    _require(x.ndim >= 2 and w_up.ndim == 2 and w_gate.ndim == 2,
             "Incorrect number of dimensions for LHS or RHS")
    D, I = _weight_dims(w_up, weights_out_in)
    # (the messages are only built when a check fails: this runs once per training step)
    if x.shape[-1] != D:
        raise ShapeError(f"Dimension mismatch. Expected x.shape[-1] ({x.shape[-1]}) to be equal to "
                         f"w_up.shape[{1 if weights_out_in else 0}] ({D})")
    _require(w_up.shape == w_gate.shape, "Expected both weight matrices to have same shape")
    if not (x.dtype == dtype and w_gate.dtype == dtype and w_up.dtype == dtype):
        raise ShapeError(f"Expected {dtype} inputs and weights, got {x.dtype}, {w_gate.dtype}, {w_up.dtype}")
    dev = x.device
    if dev.type != "cuda" or w_gate.device != dev or w_up.device != dev:
        _check_device(x, w_gate, w_up)
    _require(x.numel() > 0 and I > 0, "empty input")
    x2, wg, wu = _rows(x), _rows(w_gate), _rows(w_up)
    if _ld(wg) != _ld(wu):
        wg, wu = wg.contiguous(), wu.contiguous()
    T = x2.shape[0]
    out_shape = tuple(x.shape[:-1]) + (I,)
    out = torch.empty(out_shape, device=dev, dtype=dtype)
    g = torch.empty_like(out) if save_preactivations else None
    u = torch.empty_like(out) if save_preactivations else None
    with _on_device(dev):
        _abi.check(_abi.lib().fsw_swiglu_forward(
            x2.data_ptr(), wg.data_ptr(), wu.data_ptr(), out.data_ptr(),
            g.data_ptr() if g is not None else None, u.data_ptr() if u is not None else None,
            T, D, I, _ld(x2), _ld(wg), I, _code(dtype, weights_out_in), _stream_ptr(dev)))
    return out, g, u


def elementwise_backward(grad_output: torch.Tensor, xw_gate: torch.Tensor, xw_up: torch.Tensor,
                         dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (grad_xw_up, grad_xw_gate) -- the reference's order (kernels_bf16.py:255)."""
    _require(grad_output.shape == xw_gate.shape == xw_up.shape,
             "grad_output, xw_gate and xw_up must have the same shape")
    _require(grad_output.dtype == dtype and xw_gate.dtype == dtype and xw_up.dtype == dtype,
             f"Expected {dtype} tensors")
    dev = _check_device(grad_output, xw_gate, xw_up)
    _require(grad_output.numel() > 0, "empty input")
    # the kernel indexes flat, dense arrays (the reference silently assumes this, :224-226)
    dout, g, u = grad_output.contiguous(), xw_gate.contiguous(), xw_up.contiguous()
    grad_xw_up = torch.empty_like(dout)
    grad_xw_gate = torch.empty_like(dout)
    with _on_device(dev):
        _abi.check(_abi.lib().fsw_elementwise_backward(
            dout.data_ptr(), g.data_ptr(), u.data_ptr(), grad_xw_up.data_ptr(),
            grad_xw_gate.data_ptr(), dout.numel(), _DTYPE_CODE[dtype], _stream_ptr(dev)))
    return grad_xw_up, grad_xw_gate


def gating_grad_recompute(grad_output: torch.Tensor, x: torch.Tensor, w_gate: torch.Tensor,
                          w_up: torch.Tensor, dtype: torch.dtype,
                          weights_out_in: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(grad_xw_up, grad_xw_gate) like elementwise_backward, but from x and the weights: the
    pre-activations x@w_gate and x@w_up are recomputed in fp32 inside the kernel and never stored.
    For backward passes that did not save them (fused_swiglu/swiglu.py:28 saves them always)."""
    _require(x.ndim >= 2 and w_up.ndim == 2 and w_gate.ndim == 2,
             "Incorrect number of dimensions for LHS or RHS")
    D, I = _weight_dims(w_up, weights_out_in)
    _require(x.shape[-1] == D,
             f"Dimension mismatch. Expected x.shape[-1] ({x.shape[-1]}) to be equal to "
             f"w_up.shape[{1 if weights_out_in else 0}] ({D})")
    _require(w_up.shape == w_gate.shape, "Expected both weight matrices to have same shape")
    _require(tuple(grad_output.shape) == tuple(x.shape[:-1]) + (I,),
             f"grad_output {tuple(grad_output.shape)} does not match x {tuple(x.shape)} and I = {I}")
    _require(all(t.dtype == dtype for t in (grad_output, x, w_gate, w_up)), f"Expected {dtype} tensors")
    dev = _check_device(grad_output, x, w_gate, w_up)
    _require(x.numel() > 0 and I > 0, "empty input")
    x2, wg, wu = _rows(x), _rows(w_gate), _rows(w_up)
    if _ld(wg) != _ld(wu):
        wg, wu = wg.contiguous(), wu.contiguous()
    dout = grad_output.contiguous()
    grad_xw_up = torch.empty_like(dout)
    grad_xw_gate = torch.empty_like(dout)
    with _on_device(dev):
        _abi.check(_abi.lib().fsw_gating_grad_recompute(
            x2.data_ptr(), wg.data_ptr(), wu.data_ptr(), dout.data_ptr(), grad_xw_up.data_ptr(),
            grad_xw_gate.data_ptr(), x2.shape[0], D, I, _ld(x2), _ld(wg), I, _code(dtype, weights_out_in),
            _stream_ptr(dev)))
    return grad_xw_up, grad_xw_gate


def fused_input_grad(grad_xw_gate: torch.Tensor, grad_xw_up: torch.Tensor, w_gate: torch.Tensor,
                     w_up: torch.Tensor, dtype: torch.dtype, weights_out_in: bool = False) -> torch.Tensor:
    """grad_x = grad_xw_gate @ w_gate.T + grad_xw_up @ w_up.T in one kernel (swiglu.py:45)."""
    _require(grad_xw_gate.shape == grad_xw_up.shape, "gate/up gradient shapes differ")
    _require(w_gate.ndim == 2 and w_gate.shape == w_up.shape,
             "Expected both weight matrices to have same shape")
    D, I = _weight_dims(w_gate, weights_out_in)
    _require(grad_xw_gate.shape[-1] == I, "Dimension mismatch between gradients and weights")
    _require(all(t.dtype == dtype for t in (grad_xw_gate, grad_xw_up, w_gate, w_up)),
             f"Expected {dtype} tensors")
    dev = _check_device(grad_xw_gate, grad_xw_up, w_gate, w_up)
    dg, du, wg, wu = _rows(grad_xw_gate), _rows(grad_xw_up), _rows(w_gate), _rows(w_up)
    if _ld(dg) != _ld(du):
        dg, du = dg.contiguous(), du.contiguous()
    if _ld(wg) != _ld(wu):
        wg, wu = wg.contiguous(), wu.contiguous()
    T = dg.shape[0]
    grad_x = torch.empty(tuple(grad_xw_gate.shape[:-1]) + (D,), device=dev, dtype=dtype)
    with _on_device(dev):
        flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
        ws, ws_bytes = _workspace(_abi.STEP_INPUT_GRAD | flag, T, D, I, dev)
        _abi.check(_abi.lib().fsw_input_grad(
            dg.data_ptr(), du.data_ptr(), wg.data_ptr(), wu.data_ptr(), grad_x.data_ptr(),
            T, D, I, _ld(dg), _ld(wg), D, ws.data_ptr() if ws is not None else None, ws_bytes,
            _code(dtype, weights_out_in), _stream_ptr(dev)))
    return grad_x


def swiglu_backward(grad_output: torch.Tensor, x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
                    xw_gate: torch.Tensor, xw_up: torch.Tensor, dtype: torch.dtype, need_input_grad: bool = True,
                    need_weight_grad: bool = True, weights_out_in: bool = False
                    ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(grad_x, grad_w_gate, grad_w_up) of fused_swiglu/swiglu.py:34-58 in ONE library call: the gating gradient,
    then the input-gradient and weight-gradient GEMMs that were asked for.  Same kernels, same results as
    elementwise_backward + fused_input_grad + fused_weight_grad; two trips through ctypes and their argument checks
    fewer, which is most of a training step's host time when d_model is small."""
    D, I = _weight_dims(w_gate, weights_out_in)
    if not (x.ndim >= 2 and w_gate.ndim == 2 and w_gate.shape == w_up.shape and x.shape[-1] == D
            and xw_gate.shape == xw_up.shape == grad_output.shape and tuple(grad_output.shape) == tuple(x.shape[:-1]) + (I,)):
        raise ShapeError(f"swiglu_backward: shapes do not fit: x {tuple(x.shape)}, weights {tuple(w_gate.shape)} / "
                         f"{tuple(w_up.shape)}, pre-activations {tuple(xw_gate.shape)} / {tuple(xw_up.shape)}, "
                         f"grad_output {tuple(grad_output.shape)}")
    if not (x.dtype == w_gate.dtype == w_up.dtype == xw_gate.dtype == xw_up.dtype == grad_output.dtype == dtype):
        raise ShapeError(f"Expected {dtype} tensors")
    dev = x.device
    if dev.type != "cuda" or not (w_gate.device == w_up.device == xw_gate.device == xw_up.device == grad_output.device == dev):
        _check_device(x, w_gate, w_up, xw_gate, xw_up, grad_output)   # raises with the offending pair
    if x.numel() == 0 or I == 0:
        raise ShapeError("empty input")
    x2, wg, wu = _rows(x), _rows(w_gate), _rows(w_up)
    if _ld(wg) != _ld(wu):
        wg, wu = wg.contiguous(), wu.contiguous()
    # the gating gradient indexes flat, dense arrays
    dout, g, u = grad_output.contiguous(), xw_gate.contiguous(), xw_up.contiguous()
    T = x2.shape[0]
    grad_xw_gate, grad_xw_up = torch.empty_like(dout), torch.empty_like(dout)
    grad_x = torch.empty(x.shape, device=dev, dtype=dtype) if need_input_grad else None
    grad_w_gate = torch.empty(w_gate.shape, device=dev, dtype=dtype) if need_weight_grad else None
    grad_w_up = torch.empty(w_up.shape, device=dev, dtype=dtype) if need_weight_grad else None
    with _on_device(dev):
        L = _abi.lib()
        flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
        nbytes = max(int(L.fsw_workspace_bytes(_abi.STEP_INPUT_GRAD | flag, T, D, I)) if need_input_grad else 0,
                     int(L.fsw_workspace_bytes(_abi.STEP_WEIGHT_GRAD | flag, T, D, I)) if need_weight_grad else 0)
        ws = torch.empty(nbytes, device=dev, dtype=torch.uint8) if nbytes > 0 else None
        ld_dw = w_gate.shape[1]
        _abi.check(L.fsw_swiglu_backward(
            dout.data_ptr(), g.data_ptr(), u.data_ptr(), x2.data_ptr(), wg.data_ptr(), wu.data_ptr(),
            grad_xw_gate.data_ptr(), grad_xw_up.data_ptr(), grad_x.data_ptr() if need_input_grad else None,
            grad_w_gate.data_ptr() if need_weight_grad else None, grad_w_up.data_ptr() if need_weight_grad else None,
            T, D, I, _ld(x2), _ld(wg), D, ld_dw, ws.data_ptr() if ws is not None else None, nbytes,
            _code(dtype, weights_out_in), _stream_ptr(dev)))
    return grad_x, grad_w_gate, grad_w_up


def fused_weight_grad(x: torch.Tensor, grad_xw_up: torch.Tensor, grad_xw_gate: torch.Tensor,
                      dtype: torch.dtype,
                      out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                      weights_out_in: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """(grad_w_up, grad_w_gate) = (x^T grad_xw_up, x^T grad_xw_gate), each [D, I], reduced over
    every token in fp32.  Same argument and return order as fused_bmm (kernels_bf16.py:385-412),
    with the batch sum of swiglu.py:56-57 folded in.  `out` = (grad_w_up, grad_w_gate) lets the
    caller supply the two result arrays, e.g. the halves of one packed [D, 2I] gradient; they must
    have unit inner stride and the same row stride."""
    _require(grad_xw_up.shape == grad_xw_gate.shape, "gate/up gradient shapes differ")
    _require(x.shape[:-1] == grad_xw_up.shape[:-1],
             f"Dimension mismatch. x {tuple(x.shape)} vs gradients {tuple(grad_xw_up.shape)}")
    _require(all(t.dtype == dtype for t in (x, grad_xw_up, grad_xw_gate)), f"Expected {dtype} tensors")
    dev = _check_device(x, grad_xw_up, grad_xw_gate)
    x2, du, dg = _rows(x), _rows(grad_xw_up), _rows(grad_xw_gate)
    if _ld(dg) != _ld(du):
        dg, du = dg.contiguous(), du.contiguous()
    T, D = x2.shape
    I = du.shape[1]
    wshape = (I, D) if weights_out_in else (D, I)
    if out is None:
        grad_w_up = torch.empty(wshape, device=dev, dtype=dtype)
        grad_w_gate = torch.empty(wshape, device=dev, dtype=dtype)
    else:
        grad_w_up, grad_w_gate = out
        _require(tuple(grad_w_up.shape) == wshape and tuple(grad_w_gate.shape) == wshape,
                 f"weight-gradient outputs must be {list(wshape)}")
        _require(grad_w_up.dtype == dtype and grad_w_gate.dtype == dtype, f"Expected {dtype} tensors")
        _check_device(x, grad_w_up, grad_w_gate)
        _require(grad_w_up.stride(-1) == 1 and grad_w_gate.stride(-1) == 1 and _ld(grad_w_up) == _ld(grad_w_gate)
                 and _ld(grad_w_up) >= wshape[1],
                 "weight-gradient outputs need unit inner stride and equal row strides")
    with _on_device(dev):
        flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
        ws, ws_bytes = _workspace(_abi.STEP_WEIGHT_GRAD | flag, T, D, I, dev)
        _abi.check(_abi.lib().fsw_weight_grad(
            x2.data_ptr(), du.data_ptr(), dg.data_ptr(), grad_w_up.data_ptr(), grad_w_gate.data_ptr(),
            T, D, I, _ld(x2), _ld(du), _ld(grad_w_up), ws.data_ptr() if ws is not None else None, ws_bytes,
            _code(dtype, weights_out_in), _stream_ptr(dev)))
    return grad_w_up, grad_w_gate


# ---- the down projection that follows the SwiGLU (w_down [I, D]; [D, I] with weights_out_in) ----
def _down_dims(w_down: torch.Tensor, weights_out_in: bool) -> Tuple[int, int]:
    _require(w_down.ndim == 2, "w_down must be 2-D")
    return (w_down.shape[1], w_down.shape[0]) if weights_out_in else (w_down.shape[0], w_down.shape[1])  # (I, D)


def down_proj_forward(act: torch.Tensor, w_down: torch.Tensor, dtype: torch.dtype,
                      weights_out_in: bool = False) -> torch.Tensor:
    """y = act @ w_down (act [..., I], w_down [I, D]; act @ w_down.T for w_down [D, I])."""
    I, D = _down_dims(w_down, weights_out_in)
    _require(act.ndim >= 2 and act.shape[-1] == I, f"Dimension mismatch: act {tuple(act.shape)} vs I = {I}")
    _require(act.dtype == dtype and w_down.dtype == dtype, f"Expected {dtype} tensors")
    dev = _check_device(act, w_down)
    _require(act.numel() > 0 and D > 0, "empty input")
    a2, w2 = _rows(act), _rows(w_down)
    T = a2.shape[0]
    y = torch.empty(tuple(act.shape[:-1]) + (D,), device=dev, dtype=dtype)
    flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
    with _on_device(dev):
        ws, ws_bytes = _workspace(_abi.STEP_DOWN_FORWARD | flag, T, D, I, dev)
        _abi.check(_abi.lib().fsw_down_proj_forward(
            a2.data_ptr(), w2.data_ptr(), y.data_ptr(), T, I, D, _ld(a2), _ld(w2), D,
            ws.data_ptr() if ws is not None else None, ws_bytes, _code(dtype, weights_out_in), _stream_ptr(dev)))
    return y


def down_proj_input_grad(grad_y: torch.Tensor, w_down: torch.Tensor, dtype: torch.dtype,
                         weights_out_in: bool = False) -> torch.Tensor:
    """grad_act = grad_y @ w_down.T (grad_y [..., D])."""
    I, D = _down_dims(w_down, weights_out_in)
    _require(grad_y.ndim >= 2 and grad_y.shape[-1] == D, f"Dimension mismatch: grad_y {tuple(grad_y.shape)} vs D = {D}")
    _require(grad_y.dtype == dtype and w_down.dtype == dtype, f"Expected {dtype} tensors")
    dev = _check_device(grad_y, w_down)
    g2, w2 = _rows(grad_y), _rows(w_down)
    T = g2.shape[0]
    grad_act = torch.empty(tuple(grad_y.shape[:-1]) + (I,), device=dev, dtype=dtype)
    flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
    with _on_device(dev):
        ws, ws_bytes = _workspace(_abi.STEP_DOWN_INPUT_GRAD | flag, T, D, I, dev)
        _abi.check(_abi.lib().fsw_down_proj_input_grad(
            g2.data_ptr(), w2.data_ptr(), grad_act.data_ptr(), T, I, D, _ld(g2), _ld(w2), I,
            ws.data_ptr() if ws is not None else None, ws_bytes, _code(dtype, weights_out_in), _stream_ptr(dev)))
    return grad_act


def down_proj_weight_grad(act: torch.Tensor, grad_y: torch.Tensor, dtype: torch.dtype,
                          weights_out_in: bool = False) -> torch.Tensor:
    """grad_w_down = act^T grad_y over every token, [I, D] ([D, I] with weights_out_in), fp32 reduction."""
    _require(act.shape[:-1] == grad_y.shape[:-1], f"Dimension mismatch: act {tuple(act.shape)} vs grad_y {tuple(grad_y.shape)}")
    _require(act.dtype == dtype and grad_y.dtype == dtype, f"Expected {dtype} tensors")
    dev = _check_device(act, grad_y)
    a2, g2 = _rows(act), _rows(grad_y)
    T, I = a2.shape
    D = g2.shape[1]
    grad_w = torch.empty((D, I) if weights_out_in else (I, D), device=dev, dtype=dtype)
    flag = _abi.WEIGHTS_OUT_IN if weights_out_in else 0
    with _on_device(dev):
        ws, ws_bytes = _workspace(_abi.STEP_DOWN_WEIGHT_GRAD | flag, T, D, I, dev)
        _abi.check(_abi.lib().fsw_down_proj_weight_grad(
            a2.data_ptr(), g2.data_ptr(), grad_w.data_ptr(), T, I, D, _ld(a2), _ld(g2), grad_w.shape[1],
            ws.data_ptr() if ws is not None else None, ws_bytes, _code(dtype, weights_out_in), _stream_ptr(dev)))
    return grad_w


def fused_bmm(x_t: torch.Tensor, grad_xw_up: torch.Tensor, grad_xw_gate: torch.Tensor,
              dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """Signature-compatible with the reference's fused_bmm (kernels_bf16.py:385-412):
    x_t is the [B, D, S] view of x, the gradients are [B, S, I]; returns per-batch
    (grad_w_up, grad_w_gate) of shape [B, D, I].  The autograd Functions of this package use
    fused_weight_grad instead, which reduces over the batch inside the kernel."""
    _require(x_t.ndim == 3 and grad_xw_up.ndim == 3, "Incorrect number of dimensions for LHS or RHS")
    _require(x_t.shape[-1] == grad_xw_up.shape[-2],
             f"Dimension mismatch. Expected x.shape[2] ({x_t.shape[-1]}) to be equal to "
             f"grad.shape[1] ({grad_xw_up.shape[-2]})")
    B = x_t.shape[0]
    ups, gates = [], []
    for b in range(B):
        gu, gg = fused_weight_grad(x_t[b].transpose(0, 1), grad_xw_up[b], grad_xw_gate[b], dtype)
        ups.append(gu)
        gates.append(gg)
    return torch.stack(ups), torch.stack(gates)
