"""`nn.Module` wrapper around the fused SwiGLU path: the caller side of the operator boundary.

The reference stops at `FusedSwiGLU.apply(x, w_gate, w_up)` and leaves holding the weights to the
user (README.md:25-38).  `SwiGLU` owns them in the layout the kernels want ([d_model,
d_intermediate], unit inner stride), initialised like the reference's tests draw them
(N(0, 1)/sqrt(d_model), test_swiglu.py:30-35), either as two parameters or as one packed
[d_model, 2*d_intermediate] parameter [w_gate | w_up].  `recompute=True` keeps no pre-activations
between forward and backward (2*T*d_intermediate elements less per call) and recomputes them in the
backward's gating-gradient kernel."""
from __future__ import annotations

import torch
from torch import nn

from . import ops


class SwiGLU(nn.Module):
    def __init__(self, d_model: int, d_intermediate: int, dtype: torch.dtype = torch.bfloat16,
                 device=None, packed: bool = False, recompute: bool = False):
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float16):
            raise ValueError(f"SwiGLU computes in bfloat16 or float16, got {dtype}")
        self.d_model, self.d_intermediate, self.packed = d_model, d_intermediate, packed
        self.recompute = recompute
        kw = dict(device=device, dtype=dtype)
        if packed:
            self.w_gate_up = nn.Parameter(torch.empty(d_model, 2 * d_intermediate, **kw))
        else:
            self.w_gate = nn.Parameter(torch.empty(d_model, d_intermediate, **kw))
            self.w_up = nn.Parameter(torch.empty(d_model, d_intermediate, **kw))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        std = self.d_model ** -0.5
        for p in self.parameters():
            if p.device.type != "meta":
                nn.init.normal_(p, mean=0.0, std=std)

    @classmethod
    def from_linear(cls, gate_proj: nn.Linear, up_proj: nn.Linear, dtype: torch.dtype = None,
                    packed: bool = False, recompute: bool = False) -> "SwiGLU":
        """Build from the usual pair of bias-free `nn.Linear(d_model, d_intermediate)` projections,
        whose weights are stored [d_intermediate, d_model]: they are transposed once into the
        [d_model, d_intermediate] layout this path computes on."""
        if gate_proj.bias is not None or up_proj.bias is not None:
            raise ValueError("SwiGLU has no bias terms")
        if gate_proj.weight.shape != up_proj.weight.shape:
            raise ValueError("gate and up projections must have the same shape")
        d_int, d_model = gate_proj.weight.shape
        dtype = dtype or gate_proj.weight.dtype
        m = cls(d_model, d_int, dtype=dtype, device=gate_proj.weight.device, packed=packed, recompute=recompute)
        with torch.no_grad():
            wg, wu = gate_proj.weight.t().to(dtype), up_proj.weight.t().to(dtype)
            if packed:
                m.w_gate_up.copy_(torch.cat([wg, wu], dim=1))
            else:
                m.w_gate.copy_(wg)
                m.w_up.copy_(wu)
        return m

    def to_linear(self):
        """The inverse of from_linear: (gate_proj, up_proj) as bias-free nn.Linear modules."""
        if self.packed:
            wg, wu = self.w_gate_up[:, :self.d_intermediate], self.w_gate_up[:, self.d_intermediate:]
        else:
            wg, wu = self.w_gate, self.w_up
        out = []
        for w in (wg, wu):
            lin = nn.Linear(self.d_model, self.d_intermediate, bias=False, device=w.device, dtype=w.dtype)
            with torch.no_grad():
                lin.weight.copy_(w.t())
            out.append(lin)
        return tuple(out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        dtype = next(self.parameters()).dtype
        if self.packed:
            return ops.swiglu_packed(x, self.w_gate_up, autocast_dtype=dtype, recompute=self.recompute)
        return ops.swiglu(x, self.w_gate, self.w_up, autocast_dtype=dtype, recompute=self.recompute)

    def extra_repr(self) -> str:
        return f"d_model={self.d_model}, d_intermediate={self.d_intermediate}, packed={self.packed}, recompute={self.recompute}"
