"""`nn.Module` wrapper around the fused SwiGLU path: the caller side of the operator boundary.

The reference stops at `FusedSwiGLU.apply(x, w_gate, w_up)` and leaves holding the weights to the
user (README.md:25-38).  `SwiGLU` owns them in the layout the kernels want ([d_model,
d_intermediate], unit inner stride), initialised like the reference's tests draw them
(N(0, 1)/sqrt(d_model), test_swiglu.py:30-35), either as two parameters or as one packed
[d_model, 2*d_intermediate] parameter [w_gate | w_up].  `weights_out_in=True` stores them the way
`nn.Linear` does ([d_intermediate, d_model]; packed: [2*d_intermediate, d_model]) and the kernels read
that layout in place, so `from_linear(..., keep_layout=True)` adopts a checkpoint's tensors without a
transpose.  `recompute=True` keeps no pre-activations between forward and backward
(2*T*d_intermediate elements less per call) and recomputes them in the backward's gating-gradient
kernel.  `SwiGLUMLP` chains the down projection behind it: the whole gated MLP block on this library."""
from __future__ import annotations

import torch
from torch import nn

from . import ops


class SwiGLU(nn.Module):
    def __init__(self, d_model: int, d_intermediate: int, dtype: torch.dtype = torch.bfloat16,
                 device=None, packed: bool = False, recompute: bool = False, weights_out_in: bool = False):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"SwiGLU computes in bfloat16 or float16, got {dtype}")
        self.d_model, self.d_intermediate, self.packed = d_model, d_intermediate, packed
        self.recompute, self.weights_out_in = recompute, weights_out_in
        kw = dict(device=device, dtype=dtype)
        one = (d_intermediate, d_model) if weights_out_in else (d_model, d_intermediate)
        both = (2 * d_intermediate, d_model) if weights_out_in else (d_model, 2 * d_intermediate)
        if packed:
            self.w_gate_up = nn.Parameter(torch.empty(*both, **kw))
        else:
            self.w_gate = nn.Parameter(torch.empty(*one, **kw))
            self.w_up = nn.Parameter(torch.empty(*one, **kw))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        std = self.d_model ** -0.5
        for p in self.parameters():
            if p.device.type != "meta":
                nn.init.normal_(p, mean=0.0, std=std)

    @classmethod
    def from_linear(cls, gate_proj: nn.Linear, up_proj: nn.Linear, dtype: torch.dtype = None,
                    packed: bool = False, recompute: bool = False, keep_layout: bool = False) -> "SwiGLU":
        """Build from the usual pair of bias-free `nn.Linear(d_model, d_intermediate)` projections,
        whose weights are stored [d_intermediate, d_model].  By default they are transposed once into
        the reference's [d_model, d_intermediate] layout; with `keep_layout=True` the module computes on
        the nn.Linear layout itself, and (unless `packed` or a dtype change forces a copy) shares the
        very Parameters of the two projections."""
        if gate_proj.bias is not None or up_proj.bias is not None:
            raise ValueError("SwiGLU has no bias terms")
        if gate_proj.weight.shape != up_proj.weight.shape:
            raise ValueError("gate and up projections must have the same shape")
        d_int, d_model = gate_proj.weight.shape
        dtype = dtype or gate_proj.weight.dtype
        m = cls(d_model, d_int, dtype=dtype, device="meta", packed=packed, recompute=recompute,
                weights_out_in=keep_layout)
        dev = gate_proj.weight.device
        with torch.no_grad():
            if keep_layout:
                wg, wu = gate_proj.weight, up_proj.weight
                if packed:
                    m.w_gate_up = nn.Parameter(torch.cat([wg, wu], dim=0).to(dtype))
                elif wg.dtype == dtype and wg.is_contiguous() and wu.is_contiguous():
                    m.w_gate, m.w_up = wg, wu  # no copy: the same Parameters
                else:
                    m.w_gate, m.w_up = nn.Parameter(wg.to(dtype).contiguous()), nn.Parameter(wu.to(dtype).contiguous())
            else:
                wg, wu = gate_proj.weight.t().to(dtype), up_proj.weight.t().to(dtype)
                if packed:
                    m.w_gate_up = nn.Parameter(torch.cat([wg, wu], dim=1).contiguous())
                else:
                    m.w_gate, m.w_up = nn.Parameter(wg.contiguous()), nn.Parameter(wu.contiguous())
        assert next(m.parameters()).device == dev
        return m

    def _gate_up(self):
        if not self.packed:
            return self.w_gate, self.w_up
        I = self.d_intermediate
        if self.weights_out_in:
            return self.w_gate_up[:I], self.w_gate_up[I:]
        return self.w_gate_up[:, :I], self.w_gate_up[:, I:]

    def to_linear(self):
        """The inverse of from_linear: (gate_proj, up_proj) as bias-free nn.Linear modules."""
        out = []
        for w in self._gate_up():
            lin = nn.Linear(self.d_model, self.d_intermediate, bias=False, device=w.device, dtype=w.dtype)
            with torch.no_grad():
                lin.weight.copy_(w if self.weights_out_in else w.t())
            out.append(lin)
        return tuple(out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        dtype = next(self.parameters()).dtype
        if self.packed:
            return ops.swiglu_packed(x, self.w_gate_up, autocast_dtype=dtype, recompute=self.recompute,
                                     weights_out_in=self.weights_out_in)
        return ops.swiglu(x, self.w_gate, self.w_up, autocast_dtype=dtype, recompute=self.recompute,
                          weights_out_in=self.weights_out_in)

    def extra_repr(self) -> str:
        return (f"d_model={self.d_model}, d_intermediate={self.d_intermediate}, packed={self.packed}, "
                f"recompute={self.recompute}, weights_out_in={self.weights_out_in}")


class SwiGLUMLP(nn.Module):
    """The gated MLP block y = (silu(x Wg) * (x Wu)) W_down: the fused SwiGLU followed by the down
    projection on the same kernels.  The reference ends at the SwiGLU output and leaves the down
    projection to its caller (README.md:25-38).  w_down is [d_intermediate, d_model], or with
    `weights_out_in` [d_model, d_intermediate] like `nn.Linear(d_intermediate, d_model).weight`."""

    def __init__(self, d_model: int, d_intermediate: int, dtype: torch.dtype = torch.bfloat16, device=None,
                 packed: bool = False, recompute: bool = False, weights_out_in: bool = False):
        super().__init__()
        self.swiglu = SwiGLU(d_model, d_intermediate, dtype=dtype, device=device, packed=packed,
                             recompute=recompute, weights_out_in=weights_out_in)
        shape = (d_model, d_intermediate) if weights_out_in else (d_intermediate, d_model)
        self.w_down = nn.Parameter(torch.empty(*shape, device=device, dtype=dtype))
        self.weights_out_in = weights_out_in
        if self.w_down.device.type != "meta":
            nn.init.normal_(self.w_down, mean=0.0, std=d_intermediate ** -0.5)

    @classmethod
    def from_linear(cls, gate_proj: nn.Linear, up_proj: nn.Linear, down_proj: nn.Linear, dtype: torch.dtype = None,
                    packed: bool = False, recompute: bool = False, keep_layout: bool = True) -> "SwiGLUMLP":
        """From the three bias-free projections of a Llama-style MLP.  `keep_layout=True` (the default here)
        computes on their [out, in] weights in place."""
        if down_proj.bias is not None:
            raise ValueError("the down projection has no bias term")
        d_model, d_int = down_proj.weight.shape
        dtype = dtype or down_proj.weight.dtype
        m = cls(d_model, d_int, dtype=dtype, device="meta", packed=packed, recompute=recompute, weights_out_in=keep_layout)
        m.swiglu = SwiGLU.from_linear(gate_proj, up_proj, dtype=dtype, packed=packed, recompute=recompute,
                                      keep_layout=keep_layout)
        with torch.no_grad():
            w = down_proj.weight
            if keep_layout and w.dtype == dtype and w.is_contiguous():
                m.w_down = w
            else:
                m.w_down = nn.Parameter((w if keep_layout else w.t()).to(dtype).contiguous())
        return m

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.down_proj(self.swiglu(x), self.w_down, autocast_dtype=self.w_down.dtype,
                             weights_out_in=self.weights_out_in)
