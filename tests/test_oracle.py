"""Pins the CPU oracle (oracle/) WITHOUT a GPU.  The reference ships no golden vectors for this
path, so each oracle function is checked against something the mathematics fixes and that a
plausible mistake (dropped term, wrong sign, transposed operand, swapped return order) breaks:
  * two independent implementations agree (naive C loops vs numpy/BLAS) on ragged tiny shapes;
  * torch.autograd of the eager formula in fp64 (a library routine) gives the same gradients;
  * central finite differences of the forward give the same gradients;
  * closed forms and invariants (Wg = 0, large g, linearity, token permutation, column slices);
  * the reference's own reproducible test data: its shape grid and rel-L2 bound.
"""
import json
import os

import numpy as np
import pytest
import torch

RAGGED = [(3, 5, 7), (1, 1, 1), (33, 72, 65), (17, 40, 24), (64, 64, 128)]


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape)


def _inputs(T, D, I, seed=0):
    return (_rand((T, D), seed), _rand((D, I), seed + 1) / np.sqrt(D), _rand((D, I), seed + 2) / np.sqrt(D),
            _rand((T, I), seed + 3))


# ---- silu / silu' ----------------------------------------------------------------------------
def test_silu_closed_forms(oracle):
    from scipy.special import expit

    z = np.linspace(-30, 30, 2001)
    assert np.allclose(oracle.silu(z), z * expit(z), rtol=1e-14, atol=1e-300)
    # d/dz [z * s(z)] by an independent route: s + z s (1 - s) == s (1 + z (1 - s))
    s = expit(z)
    assert np.allclose(oracle.silu_grad(z), s * (1 + z * (1 - s)), rtol=1e-13)
    assert oracle.silu(0.0) == 0.0 and oracle.silu_grad(0.0) == 0.5
    # asymptotes
    assert abs(oracle.silu(40.0) - 40.0) < 1e-12 and abs(oracle.silu(-40.0)) < 1e-12
    assert abs(oracle.silu_grad(40.0) - 1.0) < 1e-12 and abs(oracle.silu_grad(-40.0)) < 1e-12
    # numerical derivative
    h = 1e-6
    num = (oracle.silu(z + h) - oracle.silu(z - h)) / (2 * h)
    assert np.allclose(num, oracle.silu_grad(z), atol=1e-8)
    # the global minimum of silu is at z ~ -1.2785, where silu' changes sign
    assert oracle.silu_grad(-1.2784645427610738) == pytest.approx(0.0, abs=1e-12)


def test_c_scalar_helpers_match_numpy(oracle):
    lib = oracle.c_lib()
    for z in [-20.0, -1.5, -1e-3, 0.0, 0.3, 2.0, 15.0]:
        assert lib.osw_silu(z) == pytest.approx(float(oracle.silu(z)), rel=1e-14, abs=1e-300)
        assert lib.osw_silu_grad(z) == pytest.approx(float(oracle.silu_grad(z)), rel=1e-13)


# ---- two independent implementations -------------------------------------------------------------
@pytest.mark.parametrize("T,D,I", RAGGED)
def test_c_loops_match_numpy(oracle, T, D, I):
    x, wg, wu, dout = _inputs(T, D, I)
    out_c, g_c, u_c = oracle.c_forward(x, wg, wu)
    out_n, g_n, u_n = oracle.fused_swiglu_fwd(x, wg, wu)
    for a, b in ((out_c, out_n), (g_c, g_n), (u_c, u_n)):
        assert np.allclose(a, b, rtol=1e-12, atol=1e-13)
    dx_c, dwg_c, dwu_c = oracle.c_backward(x, wg, wu, dout)
    dx_n, dwg_n, dwu_n = oracle.swiglu_backward(x, wg, wu, dout)
    for a, b in ((dx_c, dx_n), (dwg_c, dwg_n), (dwu_c, dwu_n)):
        assert np.allclose(a, b, rtol=1e-11, atol=1e-12)
    dU_c, dG_c = oracle.c_elementwise_backward(dout, g_n, u_n)
    dU_n, dG_n = oracle.elementwise_backward(dout, g_n, u_n)
    assert np.allclose(dU_c, dU_n, rtol=1e-13) and np.allclose(dG_c, dG_n, rtol=1e-13)


# ---- against torch.autograd of the eager formula (fused_swiglu/test_swiglu.py:47-55) ------------
@pytest.mark.parametrize("shape", [(2, 5, 12, 20), (1, 33, 72, 65), (3, 4, 8, 8)])
def test_backward_matches_autograd_fp64(oracle, shape):
    B, S, D, I = shape
    x = torch.randn(B, S, D, dtype=torch.float64, generator=torch.Generator().manual_seed(1), requires_grad=True)
    wg = (torch.randn(D, I, dtype=torch.float64, generator=torch.Generator().manual_seed(2)) / D ** 0.5).requires_grad_()
    wu = (torch.randn(D, I, dtype=torch.float64, generator=torch.Generator().manual_seed(3)) / D ** 0.5).requires_grad_()
    dy = torch.randn(B, S, I, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    out = torch.nn.functional.silu(torch.matmul(x, wg)) * torch.matmul(x, wu)
    out.backward(dy)
    o_out, _, _ = oracle.fused_swiglu_fwd(x.detach().numpy(), wg.detach().numpy(), wu.detach().numpy())
    dx, dwg, dwu = oracle.swiglu_backward(x.detach().numpy(), wg.detach().numpy(), wu.detach().numpy(), dy.numpy())
    assert np.allclose(o_out, out.detach().numpy(), rtol=1e-12, atol=1e-13)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-11, atol=1e-12)
    assert np.allclose(dwg, wg.grad.numpy(), rtol=1e-11, atol=1e-12)
    assert np.allclose(dwu, wu.grad.numpy(), rtol=1e-11, atol=1e-12)
    # gate and up gradients are different things: a swapped return order must not pass
    assert not np.allclose(dwg, wu.grad.numpy(), rtol=1e-3)


def test_elementwise_backward_matches_autograd(oracle):
    g = torch.randn(7, 9, dtype=torch.float64, generator=torch.Generator().manual_seed(5), requires_grad=True)
    u = torch.randn(7, 9, dtype=torch.float64, generator=torch.Generator().manual_seed(6), requires_grad=True)
    dy = torch.randn(7, 9, dtype=torch.float64, generator=torch.Generator().manual_seed(7))
    (torch.nn.functional.silu(g) * u).backward(dy)
    dU, dG = oracle.elementwise_backward(dy.numpy(), g.detach().numpy(), u.detach().numpy())
    assert np.allclose(dU, u.grad.numpy(), rtol=1e-12) and np.allclose(dG, g.grad.numpy(), rtol=1e-12)


# ---- finite differences ----------------------------------------------------------------------
def test_backward_matches_finite_differences(oracle):
    T, D, I = 4, 6, 5
    x, wg, wu, dout = _inputs(T, D, I, seed=11)

    def loss(x_, wg_, wu_):
        return float((oracle.fused_swiglu_fwd(x_, wg_, wu_)[0] * dout).sum())

    dx, dwg, dwu = oracle.swiglu_backward(x, wg, wu, dout)
    h = 1e-6
    for arr, grad, which in ((x, dx, 0), (wg, dwg, 1), (wu, dwu, 2)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            ap, am = arr.copy(), arr.copy()
            ap[idx] += h
            am[idx] -= h
            args_p = [x, wg, wu]
            args_m = [x, wg, wu]
            args_p[which], args_m[which] = ap, am
            num[idx] = (loss(*args_p) - loss(*args_m)) / (2 * h)
        assert np.allclose(num, grad, rtol=1e-6, atol=1e-8)


# ---- the down projection and the whole MLP block --------------------------------------------------
@pytest.mark.parametrize("T,D,I", RAGGED)
def test_down_proj_c_loops_match_numpy(oracle, T, D, I):
    rng = np.random.default_rng(T * 1000 + D)
    act, w, dy = rng.standard_normal((T, I)), rng.standard_normal((I, D)) / I ** 0.5, rng.standard_normal((T, D))
    y_c, da_c, dw_c = oracle.c_down_proj(act, w, dy)
    da_n, dw_n = oracle.down_proj_backward(act, w, dy)
    assert np.allclose(y_c, oracle.down_proj_fwd(act, w), rtol=1e-12, atol=1e-13)
    assert np.allclose(da_c, da_n, rtol=1e-12, atol=1e-13) and np.allclose(dw_c, dw_n, rtol=1e-12, atol=1e-13)
    assert dw_n.shape == (I, D) and da_n.shape == (T, I)


def test_mlp_block_matches_autograd_fp64_and_finite_differences(oracle):
    B, S, D, I = 2, 5, 12, 20
    gen = lambda k: torch.Generator().manual_seed(k)
    x = torch.randn(B, S, D, dtype=torch.float64, generator=gen(1), requires_grad=True)
    wg = (torch.randn(D, I, dtype=torch.float64, generator=gen(2)) / D ** 0.5).requires_grad_()
    wu = (torch.randn(D, I, dtype=torch.float64, generator=gen(3)) / D ** 0.5).requires_grad_()
    wd = (torch.randn(I, D, dtype=torch.float64, generator=gen(4)) / I ** 0.5).requires_grad_()
    dy = torch.randn(B, S, D, dtype=torch.float64, generator=gen(5))
    y = torch.matmul(torch.nn.functional.silu(torch.matmul(x, wg)) * torch.matmul(x, wu), wd)
    y.backward(dy)
    n = lambda t: t.detach().numpy()
    o_y, dx, dwg, dwu, dwd = oracle.mlp_fwd_bwd(n(x), n(wg), n(wu), n(wd), n(dy))
    assert np.allclose(o_y, n(y), rtol=1e-12, atol=1e-13)
    for got, want in ((dx, x.grad), (dwg, wg.grad), (dwu, wu.grad), (dwd, wd.grad)):
        assert np.allclose(got, want.numpy(), rtol=1e-10, atol=1e-12)
    # a transposed down weight or a dropped term must not pass: dW_down != (dy^T act)^T only by layout,
    # and the gradient w.r.t. a single element agrees with a central difference
    h, idx = 1e-6, (3, 7)
    wp, wm = n(wd).copy(), n(wd).copy()
    wp[idx] += h
    wm[idx] -= h
    loss = lambda w: float((oracle.down_proj_fwd(oracle.fused_swiglu_fwd(n(x), n(wg), n(wu))[0], w) * n(dy)).sum())
    assert abs((loss(wp) - loss(wm)) / (2 * h) - dwd[idx]) < 1e-6 * max(1.0, abs(dwd[idx]))
    # special case: an identity down weight (I == D) passes the SwiGLU output and gradient through
    sq = np.random.default_rng(0).standard_normal((6, 8))
    assert np.allclose(oracle.down_proj_fwd(sq, np.eye(8)), sq)
    da, dw = oracle.down_proj_backward(sq, np.eye(8), sq)
    assert np.allclose(da, sq) and np.allclose(dw, sq.T @ sq)


# ---- invariants and special cases --------------------------------------------------------------
def test_zero_gate_weights(oracle):
    T, D, I = 6, 8, 10
    x, _, wu, dout = _inputs(T, D, I, seed=3)
    wg = np.zeros((D, I))
    out, g, u = oracle.fused_swiglu_fwd(x, wg, wu)
    assert np.all(out == 0) and np.all(g == 0)
    dU, dG = oracle.elementwise_backward(dout, g, u)
    assert np.all(dU == 0)
    assert np.allclose(dG, dout * u * 0.5, rtol=1e-15)  # silu'(0) = 1/2


def test_large_gate_is_bilinear(oracle):
    # g >> 0  =>  silu(g) -> g, so out -> (x Wg) * (x Wu)
    T, D, I = 5, 4, 3
    x = np.abs(_rand((T, D), 1)) + 1.0
    wg = np.abs(_rand((D, I), 2)) * 20 + 20
    wu = _rand((D, I), 3)
    out, g, u = oracle.fused_swiglu_fwd(x, wg, wu)
    assert g.min() > 40
    assert np.allclose(out, g * u, rtol=1e-12)


def test_linearity_permutation_and_slices(oracle):
    B, S, D, I = 2, 6, 8, 12
    x = _rand((B, S, D), 1)
    wg, wu = _rand((D, I), 2) / np.sqrt(D), _rand((D, I), 3) / np.sqrt(D)
    d1, d2 = _rand((B, S, I), 4), _rand((B, S, I), 5)
    g1 = oracle.swiglu_backward(x, wg, wu, d1)
    g2 = oracle.swiglu_backward(x, wg, wu, d2)
    g12 = oracle.swiglu_backward(x, wg, wu, 2.0 * d1 - 3.0 * d2)
    for a, b, c in zip(g1, g2, g12):
        assert np.allclose(c, 2.0 * a - 3.0 * b, rtol=1e-11, atol=1e-12)
    # (B, S, D) is the same problem as (1, B*S, D)
    flat = oracle.swiglu_backward(x.reshape(1, B * S, D), wg, wu, d1.reshape(1, B * S, I))
    assert np.allclose(flat[0].reshape(B, S, D), g1[0]) and np.allclose(flat[1], g1[1]) and np.allclose(flat[2], g1[2])
    # permuting tokens permutes out/dx and leaves dW alone
    perm = np.random.default_rng(0).permutation(B * S)
    xp, dp = x.reshape(-1, D)[perm], d1.reshape(-1, I)[perm]
    gp = oracle.swiglu_backward(xp, wg, wu, dp)
    assert np.allclose(gp[0], g1[0].reshape(-1, D)[perm])
    assert np.allclose(gp[1], g1[1], rtol=1e-11, atol=1e-12) and np.allclose(gp[2], g1[2], rtol=1e-11, atol=1e-12)
    # column slices of the intermediate dimension are independent (tensor-parallel shards)
    out = oracle.fused_swiglu_fwd(x, wg, wu)[0]
    h = I // 2
    assert np.allclose(out[..., :h], oracle.fused_swiglu_fwd(x, wg[:, :h], wu[:, :h])[0])
    dx_a = oracle.swiglu_backward(x, wg[:, :h], wu[:, :h], d1[..., :h])[0]
    dx_b = oracle.swiglu_backward(x, wg[:, h:], wu[:, h:], d1[..., h:])[0]
    assert np.allclose(dx_a + dx_b, g1[0], rtol=1e-11, atol=1e-12)


def test_return_orders(oracle):
    """The reference's launchers return (dU, dG) and (dWu, dWg); its backward returns
    (dx, dWg, dWu) (kernels_bf16.py:255, :412; swiglu.py:54-58)."""
    x, wg, wu, dout = _inputs(5, 6, 7, seed=9)
    _, g, u = oracle.fused_swiglu_fwd(x, wg, wu)
    dU, dG = oracle.elementwise_backward(dout, g, u)
    assert np.allclose(dU, dout * oracle.silu(g))
    dWu, dWg = oracle.weight_grad(x, dU, dG)
    assert np.allclose(dWu, x.T @ dU) and np.allclose(dWg, x.T @ dG)
    dx, dWg2, dWu2 = oracle.swiglu_backward(x, wg, wu, dout)
    assert np.allclose(dWg2, dWg) and np.allclose(dWu2, dWu)
    assert np.allclose(dx, oracle.input_grad(dG, dU, wg, wu))


# ---- 16-bit rounding helpers ---------------------------------------------------------------------
def test_round_bf16_matches_torch(oracle):
    a = np.random.default_rng(0).standard_normal(10000).astype(np.float32) * 37.0
    a = np.concatenate([a, np.float32([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895e38, 1e-40])])
    ref = torch.from_numpy(a).to(torch.bfloat16).to(torch.float64).numpy()
    assert np.array_equal(oracle.round_bf16(a), ref)
    ref16 = torch.from_numpy(a).to(torch.float16).to(torch.float64).numpy()
    assert np.array_equal(oracle.round_fp16(a), ref16)


def test_reference_rounding_emulation_error_levels(oracle):
    """The emulated rounding sequence of the reference stays well inside its own 1e-2 bound, and
    the bounds this build tests against (1e-2 bf16, 5e-3 fp16) have headroom over it."""
    B, S, D, I = 2, 128, 256, 384
    for dtype, bound in (("bf16", oracle.BFLOAT16_MAX_TOL), ("fp16", oracle.FLOAT16_MAX_TOL)):
        x, wg, wu, dy = oracle.make_input_weights(B, S, D, I, seed=0, dtype=dtype, dout_scale=1.0)
        exact_out = oracle.fused_swiglu_fwd(x, wg, wu)[0]
        exact = (exact_out,) + oracle.swiglu_backward(x, wg, wu, dy)
        emu = oracle.reference_rounding_fwd_bwd(x, wg, wu, dy, dtype)
        for e, r in zip(emu, exact):
            err = oracle.rel_error(e, r)
            assert 0 < err < bound / 2


# ---- what carries over from the reference's test module ---------------------------------------------
def test_reference_shape_grid_fixture(oracle):
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "reference_shape_grid.json")) as f:
        gold = json.load(f)
    fwd, bwd = oracle.reference_shape_grid(gold["num_test"])
    assert [list(c) for c in fwd] == gold["fwd"] and [list(c) for c in bwd] == gold["bwd"]
    assert len(fwd) == 81 and len(bwd) == 81
    assert fwd[0] == (1, 256, 6656, 1408) and bwd[0] == (2, 1152, 2304, 4480)
    for b, s, d, i in fwd + bwd:
        assert 1 <= b <= 3 and s % 64 == 0 and d % 64 == 0 and i % 64 == 0
        # the reference's elementwise kernel drops a tail when numel % 128 != 0
        # (kernels_bf16.py:246); none of its own cases has one
        assert (b * s * i) % 128 == 0


def test_rel_error_metric(oracle):
    y = np.array([3.0, 4.0])
    assert oracle.rel_error(y, y) == 0.0
    assert oracle.rel_error(np.array([3.0, 4.5]), y) == pytest.approx(0.1)
    assert oracle.BFLOAT16_MAX_TOL == 1e-2
