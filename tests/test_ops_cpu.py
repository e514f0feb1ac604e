"""Host-side checks of the torch.library operators and the nn.Module wrapper that need no GPU:
shape inference of the fake implementations, parameter layout and initialisation, error behaviour."""
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

import fusedswiglu_amd as fsw
from fusedswiglu_amd.kernels import kernels_bf16


def test_fake_implementations_give_shapes_and_dtypes():
    with FakeTensorMode():
        for dtype in (torch.bfloat16, torch.float16):
            x = torch.empty(2, 5, 16, dtype=dtype, device="cuda")
            w = torch.empty(16, 24, dtype=dtype, device="cuda")
            out, g, u = torch.ops.fusedswiglu_amd.swiglu_forward(x, w, w, True)
            assert out.shape == g.shape == u.shape == (2, 5, 24) and out.dtype == dtype
            out, g, u = torch.ops.fusedswiglu_amd.swiglu_forward(x, w, w, False)
            assert out.shape == (2, 5, 24) and g.numel() == 0 and u.numel() == 0
            dx, dwg, dwu = torch.ops.fusedswiglu_amd.swiglu_backward(out, x, w, w, out, out, True, True, False, False)
            assert dx.shape == x.shape and dwg.shape == (16, 24) and dwu.numel() == 0
            dx, dw, rest = torch.ops.fusedswiglu_amd.swiglu_backward(out, x, w, w, out, out, False, True, True, True)
            assert dx.numel() == 0 and dw.shape == (16, 48) and rest.numel() == 0
            # nn.Linear-style [I, D] weights
            wt = torch.empty(24, 16, dtype=dtype, device="cuda")
            out2, g2, _ = torch.ops.fusedswiglu_amd.swiglu_forward(x, wt, wt, True, True)
            assert out2.shape == g2.shape == (2, 5, 24)
            dx, dwg, dwu = torch.ops.fusedswiglu_amd.swiglu_backward(out, x, wt, wt, out, out, True, True, True, False, True)
            assert dx.shape == x.shape and dwg.shape == dwu.shape == (24, 16)
            dx, dw, rest = torch.ops.fusedswiglu_amd.swiglu_backward(out, x, wt, wt, out, out, True, True, True, True, True)
            assert dw.shape == (48, 16) and rest.numel() == 0
            # the down projection and its gradients, both layouts of w_down
            for oi, wd_shape in ((False, (24, 16)), (True, (16, 24))):
                wd = torch.empty(*wd_shape, dtype=dtype, device="cuda")
                y = torch.ops.fusedswiglu_amd.down_proj_forward(out, wd, oi)
                assert y.shape == (2, 5, 16) and y.dtype == dtype
                da, dwd = torch.ops.fusedswiglu_amd.down_proj_backward(y, out, wd, True, True, oi)
                assert da.shape == out.shape and dwd.shape == wd_shape
                da, dwd = torch.ops.fusedswiglu_amd.down_proj_backward(y, out, wd, False, True, oi)
                assert da.numel() == 0 and dwd.shape == wd_shape


def test_module_parameters():
    m = fsw.SwiGLU(64, 96)
    assert m.w_gate.shape == m.w_up.shape == (64, 96) and m.w_gate.dtype == torch.bfloat16
    # N(0, 1)/sqrt(d_model), as the reference's tests draw the weights (test_swiglu.py:30-35)
    assert abs(float(m.w_gate.float().std()) * 8 - 1) < 0.1
    p = fsw.SwiGLU(64, 96, dtype=torch.float16, packed=True)
    assert p.w_gate_up.shape == (64, 192) and p.w_gate_up.dtype == torch.float16
    assert [n for n, _ in p.named_parameters()] == ["w_gate_up"]
    meta = fsw.SwiGLU(4096, 12288, device="meta")
    assert meta.w_up.is_meta
    with pytest.raises(ValueError):
        fsw.SwiGLU(8, 8, dtype=torch.float32)


def test_host_tensors_and_bad_shapes_are_rejected_before_any_launch():
    m = fsw.SwiGLU(16, 24)
    with pytest.raises(kernels_bf16.ShapeError, match="HIP GPU"):
        m(torch.zeros(2, 16, dtype=torch.bfloat16))
    with pytest.raises(kernels_bf16.ShapeError, match="packed weight"):
        fsw.swiglu_packed(torch.zeros(2, 16), torch.zeros(16, 25))


def test_module_from_and_to_linear():
    gate = torch.nn.Linear(32, 48, bias=False, dtype=torch.bfloat16)
    up = torch.nn.Linear(32, 48, bias=False, dtype=torch.bfloat16)
    for packed in (False, True):
        m = fsw.SwiGLU.from_linear(gate, up, packed=packed)
        assert (m.d_model, m.d_intermediate) == (32, 48)
        wg = m.w_gate_up[:, :48] if packed else m.w_gate
        wu = m.w_gate_up[:, 48:] if packed else m.w_up
        assert torch.equal(wg, gate.weight.t()) and torch.equal(wu, up.weight.t())
        g2, u2 = m.to_linear()
        assert torch.equal(g2.weight, gate.weight) and torch.equal(u2.weight, up.weight)
    with pytest.raises(ValueError):
        fsw.SwiGLU.from_linear(torch.nn.Linear(8, 8), up)


def test_module_keeps_the_linear_layout_without_copies():
    gate = torch.nn.Linear(32, 48, bias=False, dtype=torch.bfloat16)
    up = torch.nn.Linear(32, 48, bias=False, dtype=torch.bfloat16)
    down = torch.nn.Linear(48, 32, bias=False, dtype=torch.bfloat16)
    m = fsw.SwiGLU.from_linear(gate, up, keep_layout=True)
    assert m.weights_out_in and m.w_gate is gate.weight and m.w_up is up.weight  # the same Parameters
    assert (m.d_model, m.d_intermediate) == (32, 48)
    g2, u2 = m.to_linear()
    assert torch.equal(g2.weight, gate.weight) and torch.equal(u2.weight, up.weight)
    p = fsw.SwiGLU.from_linear(gate, up, keep_layout=True, packed=True)
    assert p.w_gate_up.shape == (96, 32) and torch.equal(p.w_gate_up[:48], gate.weight) and torch.equal(p.w_gate_up[48:], up.weight)
    fresh = fsw.SwiGLU(32, 48, weights_out_in=True)
    assert fresh.w_gate.shape == (48, 32)
    mlp = fsw.SwiGLUMLP.from_linear(gate, up, down)
    assert mlp.weights_out_in and mlp.w_down is down.weight and mlp.swiglu.w_gate is gate.weight
    assert sorted(n for n, _ in mlp.named_parameters()) == ["swiglu.w_gate", "swiglu.w_up", "w_down"]
    mlp2 = fsw.SwiGLUMLP.from_linear(gate, up, down, keep_layout=False)
    assert mlp2.w_down.shape == (48, 32) and torch.equal(mlp2.w_down, down.weight.t())
    assert fsw.SwiGLUMLP(32, 48).w_down.shape == (48, 32) and fsw.SwiGLUMLP(32, 48, weights_out_in=True).w_down.shape == (32, 48)
    with pytest.raises(ValueError):
        fsw.SwiGLUMLP.from_linear(gate, up, torch.nn.Linear(48, 32))
