"""bfloat16 launchers (the counterpart of fused_swiglu/kernels/kernels_bf16.py)."""
from functools import partial

import torch

from . import _launch

_DT = torch.bfloat16
ShapeError = _launch.ShapeError

fused_swiglu_fwd = partial(_launch.fused_swiglu_fwd, dtype=_DT)
elementwise_backward = partial(_launch.elementwise_backward, dtype=_DT)
gating_grad_recompute = partial(_launch.gating_grad_recompute, dtype=_DT)
fused_input_grad = partial(_launch.fused_input_grad, dtype=_DT)
fused_weight_grad = partial(_launch.fused_weight_grad, dtype=_DT)
swiglu_backward = partial(_launch.swiglu_backward, dtype=_DT)
fused_bmm = partial(_launch.fused_bmm, dtype=_DT)
