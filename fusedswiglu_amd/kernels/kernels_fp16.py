"""float16 launchers (the counterpart of fused_swiglu/kernels/kernels_fp16.py).

The reference accumulates in fp16 when `fast_accum` is set (kernels_fp16.py:69-75, the default)
and always in its weight-gradient kernel (:318-319).  CDNA4's MFMA units only accumulate in
fp32, so `fast_accum` is accepted for signature parity and ignored: results are at least as
accurate as the reference's."""
from functools import partial

import torch

from . import _launch

_DT = torch.float16
ShapeError = _launch.ShapeError


def fused_swiglu_fwd(x, w_gate, w_up, fast_accum: bool = True, save_preactivations: bool = True):
    del fast_accum  # fp32 accumulation regardless
    return _launch.fused_swiglu_fwd(x, w_gate, w_up, dtype=_DT, save_preactivations=save_preactivations)


elementwise_backward = partial(_launch.elementwise_backward, dtype=_DT)
gating_grad_recompute = partial(_launch.gating_grad_recompute, dtype=_DT)
fused_input_grad = partial(_launch.fused_input_grad, dtype=_DT)
fused_weight_grad = partial(_launch.fused_weight_grad, dtype=_DT)
swiglu_backward = partial(_launch.swiglu_backward, dtype=_DT)
fused_bmm = partial(_launch.fused_bmm, dtype=_DT)
