"""TEST INFRASTRUCTURE ONLY -- numpy restatement ("oracle") of fattorib/fusedswiglu.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import
this module; the product package never does.  It restates, on the CPU in fp64,
what the reference's Triton kernels and autograd Functions compute, one function
per reference function, each citing the lines it follows (paths relative to the
reference checkout).

Parity status: every function here is PINNED by tests/test_oracle.py against
independent evaluations -- the naive-loop C restatement (swiglu_oracle.c),
torch.autograd of the eager formula in fp64, central finite differences, and
closed-form special cases.  The reference ships no golden vectors (its tests
draw from the CUDA generator at run time); what carries over from its tests is
the shape grid, the input distributions, the rel-L2 metric and the 1e-2 bound,
restated at the bottom of this file.  Bit-exact Triton rounding is neither
reproducible off an NVIDIA GPU nor required: `reference_rounding_*` below
emulates the reference's rounding *sequence* only to calibrate tolerances.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Iterator, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


# --------------------------------------------------------------------------
# scalar helpers
# --------------------------------------------------------------------------
def sigmoid(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.float64)
    # numerically stable two-sided form
    e = np.exp(-np.abs(z))
    return np.where(z >= 0, 1.0 / (1.0 + e), e / (1.0 + e))


def silu(z: np.ndarray) -> np.ndarray:
    """fused_swiglu/kernels/kernels_bf16.py:9-11  silu(z) = z * sigmoid(z)."""
    z = np.asarray(z, dtype=np.float64)
    return z * sigmoid(z)


def silu_grad(z: np.ndarray) -> np.ndarray:
    """fused_swiglu/kernels/kernels_bf16.py:14-16  s + z*s*(1-s), s = sigmoid(z)."""
    z = np.asarray(z, dtype=np.float64)
    s = sigmoid(z)
    return s + z * s * (1.0 - s)


# --------------------------------------------------------------------------
# the path, fp64, one function per reference launcher
# --------------------------------------------------------------------------
def fused_swiglu_fwd(x, w_gate, w_up) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """fused_swiglu/kernels/kernels_bf16.py:162-206 (+ kernel :102-160) and the eager
    form at fused_swiglu/test_swiglu.py:47-55.  Returns (out, g, u), the launcher's order:
    g = x @ Wg, u = x @ Wu, out = silu(g) * u.  x [..., D]; weights [D, I]."""
    x = np.asarray(x, dtype=np.float64)
    w_gate = np.asarray(w_gate, dtype=np.float64)
    w_up = np.asarray(w_up, dtype=np.float64)
    g = x @ w_gate
    u = x @ w_up
    return silu(g) * u, g, u


def elementwise_backward(grad_output, xw_gate, xw_up) -> Tuple[np.ndarray, np.ndarray]:
    """fused_swiglu/kernels/kernels_bf16.py:236-255 (+ kernel :228-234).
    Returns (dU, dG) -- the reference's order: grad of the up pre-activation first."""
    dout = np.asarray(grad_output, dtype=np.float64)
    g = np.asarray(xw_gate, dtype=np.float64)
    u = np.asarray(xw_up, dtype=np.float64)
    return dout * silu(g), dout * u * silu_grad(g)


def input_grad(grad_xw_gate, grad_xw_up, w_gate, w_up) -> np.ndarray:
    """fused_swiglu/swiglu.py:45   dx = dG @ Wg^T + dU @ Wu^T."""
    dG = np.asarray(grad_xw_gate, dtype=np.float64)
    dU = np.asarray(grad_xw_up, dtype=np.float64)
    return dG @ np.asarray(w_gate, np.float64).T + dU @ np.asarray(w_up, np.float64).T


def weight_grad(x, grad_xw_up, grad_xw_gate) -> Tuple[np.ndarray, np.ndarray]:
    """fused_swiglu/swiglu.py:50-57: fused_bmm (kernels_bf16.py:385-412) followed by the
    batch sum (swiglu.py:11-13).  Returns (dWu, dWg) -- fused_bmm's order -- each [D, I],
    reduced over every leading (token) dimension."""
    x = np.asarray(x, dtype=np.float64)
    D = x.shape[-1]
    x2 = x.reshape(-1, D)
    dU = np.asarray(grad_xw_up, dtype=np.float64).reshape(x2.shape[0], -1)
    dG = np.asarray(grad_xw_gate, dtype=np.float64).reshape(x2.shape[0], -1)
    return x2.T @ dU, x2.T @ dG


def swiglu_backward(x, w_gate, w_up, grad_output) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """fused_swiglu/swiglu.py:34-58 (FusedSwiGLU.backward): returns (dx, dWg, dWu)."""
    _, g, u = fused_swiglu_fwd(x, w_gate, w_up)
    dU, dG = elementwise_backward(grad_output, g, u)
    dx = input_grad(dG, dU, w_gate, w_up)
    dWu, dWg = weight_grad(x, dU, dG)
    return dx, dWg, dWu


# --------------------------------------------------------------------------
# the step after the path: the down projection of the MLP block the reference's users build
# --------------------------------------------------------------------------
def down_proj_fwd(act, w_down) -> np.ndarray:
    """y = act @ W_down, act [..., I], W_down [I, D].  The reference ends at the SwiGLU output and leaves this
    multiplication to the caller (README.md:25-38: `output = FusedSwiGLU.apply(...)`); it is restated
    here because the build offers it as the next step of the path."""
    return np.asarray(act, dtype=np.float64) @ np.asarray(w_down, dtype=np.float64)


def down_proj_backward(act, w_down, grad_y) -> Tuple[np.ndarray, np.ndarray]:
    """(d_act, dW_down) of y = act @ W_down: d_act = dy @ W_down^T, dW_down = act^T @ dy summed over
    every leading (token) dimension."""
    act = np.asarray(act, dtype=np.float64)
    w = np.asarray(w_down, dtype=np.float64)
    dy = np.asarray(grad_y, dtype=np.float64)
    I = act.shape[-1]
    return dy @ w.T, act.reshape(-1, I).T @ dy.reshape(-1, dy.shape[-1])


def mlp_fwd_bwd(x, w_gate, w_up, w_down, grad_y):
    """The whole block y = (silu(x Wg) * (x Wu)) W_down and its gradients:
    returns (y, dx, dWg, dWu, dW_down), composing swiglu_backward (swiglu.py:34-58) with the down projection."""
    act = fused_swiglu_fwd(x, w_gate, w_up)[0]
    y = down_proj_fwd(act, w_down)
    d_act, dwd = down_proj_backward(act, w_down, grad_y)
    dx, dwg, dwu = swiglu_backward(x, w_gate, w_up, d_act)
    return y, dx, dwg, dwu, dwd


# --------------------------------------------------------------------------
# 16-bit rounding (numpy has no bf16) and the reference's rounding sequence
# --------------------------------------------------------------------------
def round_bf16(a) -> np.ndarray:
    """Round-to-nearest-even to bfloat16, returned as float64."""
    f = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    bits = f.view(np.uint32).astype(np.uint64)
    bias = 0x7FFF + ((bits >> 16) & 1)
    bits = ((bits + bias) & 0xFFFF0000).astype(np.uint32)
    return bits.view(np.float32).astype(np.float64)


def round_fp16(a) -> np.ndarray:
    return np.asarray(a, dtype=np.float32).astype(np.float16).astype(np.float64)


def rounder(dtype: str):
    return {"bf16": round_bf16, "fp16": round_fp16}[dtype]


def reference_rounding_fwd_bwd(x, w_gate, w_up, grad_output, dtype: str = "bf16"):
    """Emulates WHERE the reference rounds to 16 bit (not its summation order), to calibrate
    how large the reference's own error against fp64 is:
      * g, u saved rounded (kernels_bf16.py:143-144); silu(g) rounded before the multiply
        with the unrounded u accumulator, result rounded (:11,146,160);
      * backward reads the rounded g/u, rounds silu and silu' (:11,16), and forms the
        products in 16 bit (:230-231);
      * dx = two rounded GEMM results added in 16 bit (swiglu.py:45);
      * per-batch dW partials rounded, then summed and rounded (kernels_bf16.py:366-382,
        swiglu.py:56-57).
    Inputs are taken as already representable in `dtype`.  x must be [B,S,D].
    Returns (out, dx, dWg, dWu) as float64."""
    r = rounder(dtype)
    x = np.asarray(x, np.float64)
    wg = np.asarray(w_gate, np.float64)
    wu = np.asarray(w_up, np.float64)
    dout = np.asarray(grad_output, np.float64)
    g_acc = (x @ wg).astype(np.float32).astype(np.float64)
    u_acc = (x @ wu).astype(np.float32).astype(np.float64)
    g, u = r(g_acc), r(u_acc)
    out = r(u_acc * r(silu(g_acc)))
    dU = r(dout * r(silu(g)))
    dG = r(r(dout * u) * r(silu_grad(g)))
    dx = r(r(dG @ wg.T) + r(dU @ wu.T))
    xt = np.swapaxes(x, -1, -2)
    dWu = r(r(xt @ dU).sum(axis=0))
    dWg = r(r(xt @ dG).sum(axis=0))
    return out, dx, dWg, dWu


# --------------------------------------------------------------------------
# metric, distributions and shape grid restated from the reference's tests
# --------------------------------------------------------------------------
BFLOAT16_MAX_TOL = 1e-2  # fused_swiglu/test_swiglu.py:20
FLOAT16_MAX_TOL = 5e-3  # the fp16 path has no reference test; bound stated by this build


def rel_error(x, y) -> float:
    """fused_swiglu/test_swiglu.py:43-44  ||x - y|| / ||y|| (Frobenius)."""
    x = np.asarray(x, np.float64)
    y = np.asarray(y, np.float64)
    return float(np.linalg.norm((x - y).ravel()) / np.linalg.norm(y.ravel()))


def make_input_weights(bs: int, sq: int, d_model: int, d_intermediate: int, seed: int = 0,
                       dtype: str = "bf16", dout_scale: float = 0.1):
    """fused_swiglu/test_swiglu.py:23-40,98: x ~ N(0,1); Wg, Wu ~ N(0,1)/sqrt(D);
    dy = 0.1 * N(0,1); everything rounded to the 16-bit dtype.  The reference draws from the
    CUDA generator, so only the distributions carry over, not the values."""
    rng = np.random.default_rng(seed)
    r = rounder(dtype)
    x = r(rng.standard_normal((bs, sq, d_model), dtype=np.float32))
    s = 1.0 / math.sqrt(d_model)
    wg = r(r(rng.standard_normal((d_model, d_intermediate), dtype=np.float32)) * s)
    wu = r(r(rng.standard_normal((d_model, d_intermediate), dtype=np.float32)) * s)
    dy = r(dout_scale * rng.standard_normal((bs, sq, d_intermediate), dtype=np.float32))
    return x, wg, wu, dy


def reference_shape_grid(num_test: int = 3) -> Tuple[list, list]:
    """The 81 forward and 81 backward (B,S,D,I) cases of fused_swiglu/test_swiglu.py:58-67 and
    :81-90.  They come from numpy's legacy generator seeded with 0 (:11), drawn at import in
    this nesting order, so they are reproducible on any machine."""
    rs = np.random.RandomState(0)

    def grid() -> list:
        return [
            (int(b), int(sq), int(dm), int(di))
            for b in rs.randint(1, 4, size=num_test)
            for sq in 64 * rs.randint(1, 32, size=num_test)
            for dm in 64 * rs.randint(1, 128, size=num_test)
            for di in 64 * rs.randint(1, 128, size=num_test)
        ]

    fwd = grid()
    bwd = grid()
    return fwd, bwd


# --------------------------------------------------------------------------
# eager fp32 SwiGLU on the host cores: the timed CPU baseline
# --------------------------------------------------------------------------
def eager_torch_fwd_bwd(x, w_gate, w_up, grad_output):
    """fused_swiglu/test_swiglu.py:47-55 and :96-104 on CPU torch tensors (fp32): eager
    out = silu(x@Wg) * (x@Wu) and autograd backward.  Returns (out, dx, dWg, dWu)."""
    import torch

    x = x.detach().clone().requires_grad_(True)
    wg = w_gate.detach().clone().requires_grad_(True)
    wu = w_up.detach().clone().requires_grad_(True)
    out = torch.nn.functional.silu(torch.matmul(x, wg)) * torch.matmul(x, wu)
    out.backward(grad_output)
    return out.detach(), x.grad, wg.grad, wu.grad


# --------------------------------------------------------------------------
# ctypes view of the naive-loop C restatement (swiglu_oracle.c)
# --------------------------------------------------------------------------
_C_LIB = None


def c_library_path() -> str:
    return os.path.join(_HERE, "libswiglu_oracle.so")


def c_lib():
    global _C_LIB
    if _C_LIB is None:
        lib = ctypes.CDLL(c_library_path())
        dp = ctypes.POINTER(ctypes.c_double)
        i64 = ctypes.c_int64
        lib.osw_silu.restype = ctypes.c_double
        lib.osw_silu.argtypes = [ctypes.c_double]
        lib.osw_silu_grad.restype = ctypes.c_double
        lib.osw_silu_grad.argtypes = [ctypes.c_double]
        lib.osw_forward.argtypes = [dp, dp, dp, i64, i64, i64, dp, dp, dp]
        lib.osw_elementwise_backward.argtypes = [dp, dp, dp, i64, dp, dp]
        lib.osw_input_grad.argtypes = [dp, dp, dp, dp, i64, i64, i64, dp]
        lib.osw_weight_grad.argtypes = [dp, dp, dp, i64, i64, i64, dp, dp]
        lib.osw_backward.argtypes = [dp, dp, dp, dp, i64, i64, i64, dp, dp, dp, dp]
        lib.osw_down_proj_forward.argtypes = [dp, dp, i64, i64, i64, dp]
        lib.osw_down_proj_backward.argtypes = [dp, dp, dp, i64, i64, i64, dp, dp]
        for f in ("osw_forward", "osw_elementwise_backward", "osw_input_grad", "osw_weight_grad",
                  "osw_backward", "osw_down_proj_forward", "osw_down_proj_backward"):
            getattr(lib, f).restype = None
        _C_LIB = lib
    return _C_LIB


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _c64(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def c_forward(x, w_gate, w_up):
    """Naive-loop forward; x [T,D].  Returns (out, g, u)."""
    x, wg, wu = _c64(x), _c64(w_gate), _c64(w_up)
    T, D = x.shape
    I = wg.shape[1]
    g, u, out = (np.empty((T, I)) for _ in range(3))
    c_lib().osw_forward(_p(x), _p(wg), _p(wu), T, D, I, _p(g), _p(u), _p(out))
    return out, g, u


def c_backward(x, w_gate, w_up, grad_output):
    """Naive-loop backward; x [T,D], grad_output [T,I].  Returns (dx, dWg, dWu)."""
    x, wg, wu, dout = _c64(x), _c64(w_gate), _c64(w_up), _c64(grad_output)
    T, D = x.shape
    I = wg.shape[1]
    scratch = np.empty(4 * T * I)
    dx, dWg, dWu = np.empty((T, D)), np.empty((D, I)), np.empty((D, I))
    c_lib().osw_backward(_p(x), _p(wg), _p(wu), _p(dout), T, D, I, _p(scratch), _p(dx), _p(dWg),
                         _p(dWu))
    return dx, dWg, dWu


def c_elementwise_backward(grad_output, xw_gate, xw_up):
    """Returns (dU, dG) like the reference launcher."""
    dout, g, u = _c64(grad_output), _c64(xw_gate), _c64(xw_up)
    dU, dG = np.empty_like(dout), np.empty_like(dout)
    c_lib().osw_elementwise_backward(_p(dout), _p(g), _p(u), dout.size, _p(dU), _p(dG))
    return dU, dG


def c_down_proj(act, w_down, grad_y):
    """Naive-loop down projection; act [T,I], w_down [I,D], grad_y [T,D].  Returns (y, d_act, dW_down)."""
    act, w, dy = _c64(act), _c64(w_down), _c64(grad_y)
    T, I = act.shape
    D = w.shape[1]
    y, d_act, dw = np.empty((T, D)), np.empty((T, I)), np.empty((I, D))
    c_lib().osw_down_proj_forward(_p(act), _p(w), T, I, D, _p(y))
    c_lib().osw_down_proj_backward(_p(act), _p(w), _p(dy), T, I, D, _p(d_act), _p(dw))
    return y, d_act, dw
