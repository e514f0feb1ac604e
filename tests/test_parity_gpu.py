"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same seeded
inputs.  Metric and bounds follow the reference's test module (fused_swiglu/test_swiglu.py:20,
:43-44): relative Frobenius error, <= 1e-2 for bfloat16; the fp16 path (untested upstream) is held
to <= 5e-3.  Full-size configurations are checked on slices the oracle can afford: whole token rows
of out/dx and whole columns of the weight gradients, which the oracle computes exactly from the
matching slices of the inputs."""
import json
import os

import numpy as np
import pytest
import torch

from fusedswiglu_amd import FastAccumFusedSwiGLU, FusedSwiGLU, _abi
from fusedswiglu_amd.kernels import kernels_bf16, kernels_fp16

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.bfloat16: 1e-2, torch.float16: 5e-3}  # rel-L2 bounds (bf16: test_swiglu.py:20)
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}
FUNC = {torch.bfloat16: FusedSwiGLU, torch.float16: FastAccumFusedSwiGLU}
KERN = {torch.bfloat16: kernels_bf16, torch.float16: kernels_fp16}
try:
    # the upstream knob (test_swiglu.py:13-16), kept as an optional reducer: NUM_TEST=2 runs 16 + 16 of the
    # reference's 81 + 81 cases.  The default runs all of them, in both element types.
    NUM_TEST = int(os.environ["NUM_TEST"])
except Exception:
    NUM_TEST = None


def np64(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().double().numpy()


def dev(a: np.ndarray, dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def make(oracle, shape, dtype, seed=0, dout_scale=0.1):
    """Oracle-side inputs (float64 arrays holding values representable in `dtype`) and their
    device copies."""
    B, S, D, I = shape
    x, wg, wu, dy = oracle.make_input_weights(B, S, D, I, seed=seed, dtype=NAME[dtype], dout_scale=dout_scale)
    return (x, wg, wu, dy), tuple(dev(a, dtype) for a in (x, wg, wu, dy))


def run_fwd_bwd(dtype, tx, twg, twu, tdy):
    tx = tx.detach().clone().requires_grad_(True)
    twg = twg.detach().clone().requires_grad_(True)
    twu = twu.detach().clone().requires_grad_(True)
    out = FUNC[dtype].apply(tx, twg, twu)
    out.backward(tdy)
    torch.cuda.synchronize()
    return out.detach(), tx.grad, twg.grad, twu.grad


SMALL = [
    (1, 256, 256, 512),    # one full tile each way
    (2, 64, 128, 192),     # smaller than a tile
    (1, 520, 264, 392),    # multiples of 8 only: edge tiles in every dimension
    (3, 100, 1032, 776),
    (1, 7, 8, 8),          # tiny
    (2, 33, 72, 65),       # I not a multiple of 8 -> edge-shape kernel
    (1, 257, 100, 130),    # nothing aligned
    (1, 1, 4096, 24),      # single token, deep reduction
    (4, 512, 256, 768),    # few output tiles, long reductions: gradient GEMMs split their reduction
    (4, 500, 264, 776),    # the same with ragged edges; dx's second pass starts inside a split
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", SMALL, ids=lambda s: "x".join(map(str, s)))
def test_forward_backward_parity_small(oracle, dtype, shape):
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype)
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    o_out, _, _ = oracle.fused_swiglu_fwd(x, wg, wu)
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dy)
    tol = TOL[dtype]
    assert out.shape == tx.shape[:-1] + (shape[3],) and out.dtype == dtype
    assert dx.shape == tx.shape and dwg.shape == twg.shape and dwu.shape == twu.shape
    assert oracle.rel_error(np64(out), o_out) < tol
    assert oracle.rel_error(np64(dx), o_dx) < tol
    assert oracle.rel_error(np64(dwg), o_dwg) < tol
    assert oracle.rel_error(np64(dwu), o_dwu) < tol
    # gate/up must not be swapped: the two weight gradients differ by far more than the bound
    assert oracle.rel_error(np64(dwg), o_dwu) > 0.1


def _random_shapes(n, seed):
    """Seeded mix of shapes: 8-aligned ones (tiled kernels, ragged tile edges, split reductions,
    the weight-streaming forward for few tokens) and unaligned ones (edge-shape kernels)."""
    rng = np.random.default_rng(seed)
    shapes = []
    for i in range(n):
        B = int(rng.integers(1, 4))
        S = int(rng.choice([1, 3, 17, 64, 100, 255, 256, 300, 513]))
        if i % 3 == 2:
            D, I = int(rng.integers(1, 300)), int(rng.integers(1, 400))
        else:
            D, I = 8 * int(rng.integers(1, 140)), 8 * int(rng.integers(1, 140))
        shapes.append((B, S, D, I))
    return shapes


@pytest.mark.parametrize("shape", _random_shapes(24, seed=2024), ids=lambda s: "x".join(map(str, s)))
def test_forward_backward_parity_random_shapes(oracle, shape):
    dtype = torch.bfloat16 if (shape[1] + shape[3]) % 2 == 0 else torch.float16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype, seed=shape[2])
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    o_out, _, _ = oracle.fused_swiglu_fwd(x, wg, wu)
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dy)
    tol = TOL[dtype]
    for got, want in ((out, o_out), (dx, o_dx), (dwg, o_dwg), (dwu, o_dwu)):
        assert torch.isfinite(got).all()
        assert oracle.rel_error(np64(got), want) < tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_launchers_match_oracle_and_reference_orders(oracle, dtype):
    """Each launcher on its own, including the saved pre-activations and the (up, gate) return
    orders of the reference launchers (kernels_bf16.py:255, :412)."""
    k = KERN[dtype]
    shape = (2, 96, 160, 264)
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype, seed=3)
    out, g, u = k.fused_swiglu_fwd(tx, twg, twu)
    o_out, o_g, o_u = oracle.fused_swiglu_fwd(x, wg, wu)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(g), o_g) < tol and oracle.rel_error(np64(u), o_u) < tol
    assert oracle.rel_error(np64(out), o_out) < tol
    # elementwise step on the device's own (rounded) g, u
    dU, dG = k.elementwise_backward(tdy, g, u)
    o_dU, o_dG = oracle.elementwise_backward(dy, np64(g), np64(u))
    assert oracle.rel_error(np64(dU), o_dU) < tol and oracle.rel_error(np64(dG), o_dG) < tol
    dx = k.fused_input_grad(dG, dU, twg, twu)
    assert oracle.rel_error(np64(dx), oracle.input_grad(np64(dG), np64(dU), wg, wu)) < tol
    dWu, dWg = k.fused_weight_grad(tx, dU, dG)
    o_dWu, o_dWg = oracle.weight_grad(x, np64(dU), np64(dG))
    assert oracle.rel_error(np64(dWu), o_dWu) < tol and oracle.rel_error(np64(dWg), o_dWg) < tol
    # the reference-shaped per-batch launcher: [B, D, S] view in, [B, D, I] partials out
    pu, pg = k.fused_bmm(tx.transpose(1, 2), dU, dG)
    assert pu.shape == (shape[0], shape[2], shape[3])
    assert oracle.rel_error(np64(pu).sum(0), o_dWu) < tol and oracle.rel_error(np64(pg).sum(0), o_dWg) < tol


def test_not_worse_than_reference_rounding(oracle):
    """north star: error no worse than the reference kernel's own error against an exact CPU
    result.  The reference's rounding sequence is emulated on the CPU (oracle.reference_rounding_*)."""
    for dtype in (torch.bfloat16, torch.float16):
        shape = (2, 256, 512, 768)
        (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype, seed=1, dout_scale=1.0)
        got = run_fwd_bwd(dtype, tx, twg, twu, tdy)
        exact = (oracle.fused_swiglu_fwd(x, wg, wu)[0],) + oracle.swiglu_backward(x, wg, wu, dy)
        emu = oracle.reference_rounding_fwd_bwd(x, wg, wu, dy, NAME[dtype])
        for name, a, e, r in zip(("out", "dx", "dWg", "dWu"), got, exact, emu):
            mine, ref = oracle.rel_error(np64(a), e), oracle.rel_error(r, e)
            assert mine <= 1.05 * ref, f"{NAME[dtype]} {name}: {mine:.3e} vs reference-style {ref:.3e}"


def _grid_cases(kind):
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "reference_shape_grid.json")) as f:
        cases = json.load(f)[kind]
    if NUM_TEST is None:
        return [tuple(c) for c in cases]
    # NUM_TEST**4 cases spread over the 81, as upstream's four nested draws would give
    n = max(1, min(len(cases), NUM_TEST ** 4))
    idx = np.linspace(0, len(cases) - 1, n).round().astype(int)
    return [tuple(cases[i]) for i in idx]


def _slice_check(oracle, dtype, tx, twg, twu, tdy, out, dx, dwg, dwu, n_rows=6, n_cols=6, seed=0):
    """Oracle comparison on whole token rows (out, dx) and whole weight-gradient columns."""
    rng = np.random.default_rng(seed)
    D, I = twg.shape
    x2, dy2 = tx.reshape(-1, D), tdy.reshape(-1, I) if tdy is not None else None
    T = x2.shape[0]
    rows = np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, n_rows)]))
    cols = np.unique(np.concatenate([[0, I - 1], rng.integers(0, I, n_cols)]))
    tol = TOL[dtype]
    r_t = torch.from_numpy(rows).to(DEV)
    c_t = torch.from_numpy(cols).to(DEV)
    wg64, wu64 = np64(twg), np64(twu)
    xr = np64(x2[r_t])
    errs = {}
    errs["out"] = oracle.rel_error(np64(out.reshape(-1, I)[r_t]), oracle.fused_swiglu_fwd(xr, wg64, wu64)[0])
    if dx is not None:
        o_dx = oracle.swiglu_backward(xr, wg64, wu64, np64(dy2[r_t]))[0]
        errs["dx"] = oracle.rel_error(np64(dx.reshape(-1, D)[r_t]), o_dx)
        x64 = np64(x2)
        _, o_dwg, o_dwu = oracle.swiglu_backward(x64, wg64[:, cols], wu64[:, cols], np64(dy2[:, c_t]))
        errs["dWg"] = oracle.rel_error(np64(dwg[:, c_t]), o_dwg)
        errs["dWu"] = oracle.rel_error(np64(dwu[:, c_t]), o_dwu)
    for k, v in errs.items():
        assert v < tol, f"{k}: rel-L2 {v:.3e} >= {tol}"
    return errs


def _grid_id(case):
    return f"{case[0]:02d}-" + "x".join(map(str, case[1]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", list(enumerate(_grid_cases("fwd"))), ids=_grid_id)
def test_reference_grid_forward(oracle, case, dtype):
    """The forward cases of the reference's test (test_swiglu.py:58-78) under no_grad: all 81 shapes, in bf16
    through FusedSwiGLU as upstream and in fp16 through FastAccumFusedSwiGLU (untested upstream)."""
    B, S, D, I = case[1]
    g = torch.Generator(device=DEV).manual_seed(case[0])
    tx = torch.randn(B, S, D, device=DEV, dtype=dtype, generator=g)
    twg = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    twu = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    with torch.no_grad():
        out = FUNC[dtype].apply(tx, twg, twu)
    _slice_check(oracle, dtype, tx, twg, twu, None, out, None, None, None, n_rows=3, seed=case[0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", list(enumerate(_grid_cases("bwd"))), ids=_grid_id)
def test_reference_grid_backward(oracle, case, dtype):
    """The backward cases of the reference's test (test_swiglu.py:81-114), dy = 0.1 * randn: all 81 shapes in
    both element types; out, dx, dWg and dWu are each held to the bound."""
    B, S, D, I = case[1]
    g = torch.Generator(device=DEV).manual_seed(case[0])
    tx = torch.randn(B, S, D, device=DEV, dtype=dtype, generator=g)
    twg = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    twu = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    tdy = 0.1 * torch.randn(B, S, I, device=DEV, dtype=dtype, generator=g)
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    _slice_check(oracle, dtype, tx, twg, twu, tdy, out, dx, dwg, dwu, n_rows=3, n_cols=3, seed=case[0])


FULL = {
    "C2-bf16-4x2048x4096x12288": (torch.bfloat16, (4, 2048, 4096), 12288),
    "C3-fp16-2x4096x4096x11008": (torch.float16, (2, 4096, 4096), 11008),
}


@pytest.mark.parametrize("name", list(FULL), ids=list(FULL))
def test_full_size_configs(oracle, name):
    """The benchmark configurations at their real sizes: x ~ N(0,1), W ~ N(0,1/D), dout ~ N(0,1)."""
    dtype, xs, I = FULL[name]
    D = xs[-1]
    g = torch.Generator(device=DEV).manual_seed(0)
    tx = torch.randn(*xs, device=DEV, dtype=torch.float32, generator=g).to(dtype)
    twg = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    twu = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    tdy = torch.randn(*xs[:-1], I, device=DEV, dtype=torch.float32, generator=g).to(dtype)
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    assert torch.isfinite(out).all() and torch.isfinite(dx).all() and torch.isfinite(dwg).all()
    _slice_check(oracle, dtype, tx, twg, twu, tdy, out, dx, dwg, dwu, n_rows=4, n_cols=4)
    # size-independent properties: deterministic, and linear in the upstream gradient
    out2, dx2, dwg2, dwu2 = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    assert torch.equal(out, out2) and torch.equal(dx, dx2) and torch.equal(dwg, dwg2) and torch.equal(dwu, dwu2)
    _, dxh, dwgh, _ = run_fwd_bwd(dtype, tx, twg, twu, tdy * 0.5)
    if dtype == torch.bfloat16:
        # scaling by a power of two is exact in bf16 (fp32's exponent range, no subnormals in play)
        assert torch.equal(dxh.float() * 2, dx.float()) and torch.equal(dwgh.float() * 2, dwg.float())
    else:
        # fp16 intermediates below 2^-14 are subnormal, so halving is exact only up to their spacing
        assert float((dxh.float() * 2 - dx.float()).norm() / dx.float().norm()) < 1e-3
        assert float((dwgh.float() * 2 - dwg.float()).norm() / dwg.float().norm()) < 1e-3


@pytest.mark.parametrize("M", [16, 64, 256])
def test_skinny_forward_full_width(oracle, M):
    """Weight-streaming forward (x [M, 8192], W [8192, 28672]), 2-D input, no pre-activations."""
    D, I = 8192, 28672
    g = torch.Generator(device=DEV).manual_seed(M)
    tx = torch.randn(M, D, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    twg = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(torch.bfloat16)
    twu = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(torch.bfloat16)
    with torch.no_grad():
        out = FusedSwiGLU.apply(tx, twg, twu)
    assert out.shape == (M, I)
    _slice_check(oracle, torch.bfloat16, tx, twg, twu, None, out, None, None, None, n_rows=6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("T,D,I", [(16, 256, 30720), (33, 264, 28672), (64, 512, 26632), (5, 136, 1800), (64, 128, 128),
                                   (100, 264, 1800), (128, 256, 1024), (200, 136, 776), (256, 512, 2056), (255, 4096, 136)])
def test_skinny_forward_column_blocks(oracle, dtype, T, D, I):
    """Up to 256 tokens: the weight-streaming forward (row-count variants 32/64/128/256) gives each
    workgroup a block of 128 columns; every column of out and of the saved pre-activations must land in its place, also in a
    ragged last block and with more blocks than CUs."""
    (x, wg, wu, _), (tx, twg, twu, _) = make(oracle, (1, T, D, I), dtype, seed=T)
    out, g, u = KERN[dtype].fused_swiglu_fwd(tx, twg, twu)
    torch.cuda.synchronize()
    o_out, o_g, o_u = oracle.fused_swiglu_fwd(x, wg, wu)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(out), o_out) < tol
    assert oracle.rel_error(np64(g), o_g) < tol and oracle.rel_error(np64(u), o_u) < tol
    # per-column check: a misplaced block would hide in a whole-array norm only if it were tiny
    col_err = np.linalg.norm(np64(out)[0] - o_out[0], axis=0) / (np.linalg.norm(o_out[0], axis=0) + 1e-30)
    assert col_err.max() < 20 * tol


def test_large_config_slices(oracle):
    """x [8,4096,8192], W [8192,28672] (32768 tokens): forward + backward, checked on slices."""
    dtype, B, S, D, I = torch.bfloat16, 8, 4096, 8192, 28672
    g = torch.Generator(device=DEV).manual_seed(5)
    tx = torch.randn(B, S, D, device=DEV, dtype=dtype, generator=g)
    twg = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    twu = torch.randn(D, I, device=DEV, dtype=dtype, generator=g) / D ** 0.5
    tdy = torch.randn(B, S, I, device=DEV, dtype=dtype, generator=g)
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    _slice_check(oracle, dtype, tx, twg, twu, tdy, out, dx, dwg, dwu, n_rows=2, n_cols=2)


@pytest.mark.parametrize("shape", [(1, 100000, 512, 1536),    # very many tokens: 391 tile rows, long dW reduction
                                   (1, 520, 32768, 256),      # very deep forward reduction, split dx/dW
                                   (1, 16, 2097144, 8),       # leading dimension just under the 2^21 limit of the tiled kernels
                                   (1, 40, 8, 131072),        # one reduction step, very wide
                                   (1, 70000, 8, 8)],         # tiny matrices, many tokens
                         ids=lambda s: "x".join(map(str, s)))
def test_extreme_aspect_ratios(oracle, shape):
    """Shapes at the corners of what the tiled kernels accept, checked on slices."""
    dtype = torch.bfloat16
    B, S, D, I = shape
    g = torch.Generator(device=DEV).manual_seed(S)
    tx = torch.randn(B, S, D, device=DEV, dtype=torch.float32, generator=g).to(dtype)
    twg = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    twu = (torch.randn(D, I, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    tdy = torch.randn(B, S, I, device=DEV, dtype=torch.float32, generator=g).to(dtype)
    # forward: the weight-streaming kernel up to 128 tokens (code 2), the tiled one beyond; gradients: tiled
    assert _abi.lib().fsw_uses_tiled_kernel(0, B * S, D, I, D, I, I, I, 16) == (2 if B * S <= 128 else 1)
    assert _abi.lib().fsw_uses_tiled_kernel(1, B * S, D, I, D, I, I, D, 16) == 1
    assert _abi.lib().fsw_uses_tiled_kernel(2, B * S, D, I, D, I, I, I, 16) == 1
    out, dx, dwg, dwu = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    for t in (out, dx, dwg, dwu):
        assert torch.isfinite(t).all()
    _slice_check(oracle, dtype, tx, twg, twu, tdy, out, dx, dwg, dwu, n_rows=3, n_cols=3)


# ---- boundary behaviour ---------------------------------------------------------------------------
def _misaligned(t):
    """The same values in storage that starts 2 bytes off a 16-byte boundary: such operands take the
    edge-shape kernels (the tiled ones need 16-byte aligned pointers)."""
    buf = torch.empty(t.numel() + 8, dtype=t.dtype, device=t.device)
    view = buf[1:1 + t.numel()].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 == 2 and view.is_contiguous()
    return view


def test_edge_kernels_agree_with_tiled_kernels(oracle):
    """An aligned problem on the tiled kernels and, from misaligned copies of the same operands, on the
    edge-shape kernels: both paths meet the oracle and each other."""
    dtype, shape = torch.bfloat16, (2, 136, 264, 520)
    B, S, D, I = shape
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype, seed=7)
    assert _abi.lib().fsw_uses_tiled_kernel(0, B * S, D, I, D, I, I, I, 16) == 1
    assert _abi.lib().fsw_uses_tiled_kernel(0, B * S, D, I, D, I, I, I, 2) == 0
    tiled = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    edge = run_fwd_bwd(dtype, _misaligned(tx), _misaligned(twg), _misaligned(twu), _misaligned(tdy))
    exact = (oracle.fused_swiglu_fwd(x, wg, wu)[0],) + oracle.swiglu_backward(x, wg, wu, dy)
    for a, b, e in zip(tiled, edge, exact):
        assert oracle.rel_error(np64(a), e) < TOL[dtype] and oracle.rel_error(np64(b), e) < TOL[dtype]
        assert oracle.rel_error(np64(a), np64(b)) < TOL[dtype]


@pytest.mark.parametrize("numel", [1, 7, 127, 128, 1000, 128 * 1024 + 5])
def test_elementwise_backward_tails(oracle, numel):
    """Any element count is fully written: the reference's floor-division grid
    (kernels_bf16.py:246) would leave numel % 128 trailing elements untouched."""
    rng = np.random.default_rng(numel)
    for dtype in (torch.bfloat16, torch.float16):
        r = oracle.rounder(NAME[dtype])
        g, u, dy = (r(rng.standard_normal(numel) * s) for s in (3.0, 1.0, 1.0))
        g[: min(numel, 4)] = r(np.array([0.0, 30.0, -30.0, -1.2785])[: min(numel, 4)])
        tg, tu, tdy = dev(g, dtype), dev(u, dtype), dev(dy, dtype)
        dU, dG = KERN[dtype].elementwise_backward(tdy, tg, tu)
        o_dU, o_dG = oracle.elementwise_backward(dy, g, u)
        assert np.allclose(np64(dU), o_dU, rtol=2 ** -8 if dtype == torch.bfloat16 else 2 ** -10, atol=1e-6)
        assert np.allclose(np64(dG), o_dG, rtol=2 ** -8 if dtype == torch.bfloat16 else 2 ** -10, atol=1e-4)
    # a misaligned (offset by one element) view exercises the scalar path
    if numel > 8:
        dU2, dG2 = kernels_bf16.elementwise_backward(dev(dy, torch.bfloat16)[1:], dev(g, torch.bfloat16)[1:], dev(u, torch.bfloat16)[1:])
        o_dU, o_dG = oracle.elementwise_backward(oracle.round_bf16(dy)[1:], oracle.round_bf16(g)[1:], oracle.round_bf16(u)[1:])
        assert np.allclose(np64(dU2), o_dU, rtol=2 ** -8, atol=1e-6)


def test_noncontiguous_and_nd_inputs(oracle):
    dtype = torch.bfloat16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, (2, 48, 64, 96), dtype, seed=2)
    ref = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    # 2-D and 4-D x (the reference only takes 3-D, kernels_bf16.py:178-180)
    out2 = FusedSwiGLU.apply(tx.reshape(96, 64), twg, twu)
    assert out2.shape == (96, 96) and torch.equal(out2, ref[0].reshape(96, 96))
    out4 = FusedSwiGLU.apply(tx.reshape(2, 4, 12, 64), twg, twu)
    assert out4.shape == (2, 4, 12, 96) and torch.equal(out4.reshape(2, 48, 96), ref[0])
    # strided x, transposed-storage weights, strided upstream gradient
    xw = torch.zeros(2, 48, 128, device=DEV, dtype=dtype)
    xw[..., :64] = tx
    x_nc = xw[..., :64]
    wg_nc = twg.t().contiguous().t()
    dy_nc = tdy.transpose(0, 1).contiguous().transpose(0, 1)
    assert not x_nc.is_contiguous() and not wg_nc.is_contiguous() and not dy_nc.is_contiguous()
    got = run_fwd_bwd(dtype, x_nc, wg_nc, twu, dy_nc)
    for a, b in zip(got, ref):
        assert torch.equal(a, b)


def test_needs_input_grad_subsets_and_no_grad(oracle):
    dtype = torch.float16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, (1, 64, 64, 128), dtype, seed=4)
    full = run_fwd_bwd(dtype, tx, twg, twu, tdy)
    # only x needs a gradient
    xa = tx.clone().requires_grad_(True)
    out = FastAccumFusedSwiGLU.apply(xa, twg, twu)
    out.backward(tdy)
    assert torch.equal(xa.grad, full[1]) and twg.grad is None
    # only w_up needs a gradient
    wua = twu.clone().requires_grad_(True)
    FastAccumFusedSwiGLU.apply(tx, twg, wua).backward(tdy)
    assert torch.equal(wua.grad, full[3])
    # no_grad: same numbers, no graph
    with torch.no_grad():
        o = FastAccumFusedSwiGLU.apply(tx.clone().requires_grad_(True), twg, twu)
    assert not o.requires_grad and torch.equal(o, full[0])


def test_autocast_casts_inputs(oracle):
    """custom_fwd(cast_inputs=...) semantics of fused_swiglu/swiglu.py:18: fp32 inputs are cast
    under autocast; outside autocast a wrong dtype is an error."""
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, (1, 32, 64, 64), torch.bfloat16, seed=6)
    ref = FusedSwiGLU.apply(tx, twg, twu)
    x32 = tx.float().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = FusedSwiGLU.apply(x32, twg.float(), twu.float())
        out_ng = None
        with torch.no_grad():
            out_ng = FusedSwiGLU.apply(tx.float(), twg.float(), twu.float())
    assert out.dtype == torch.bfloat16 and torch.equal(out, ref) and torch.equal(out_ng, ref)
    out.backward(tdy)
    assert x32.grad is not None and x32.grad.dtype == torch.float32
    with pytest.raises(AssertionError):
        FusedSwiGLU.apply(tx.float(), twg.float(), twu.float())


def test_stream_and_thread_safety(oracle):
    """Launches go to the caller's current stream and the library keeps no state between calls."""
    dtype = torch.bfloat16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, (1, 128, 128, 256), dtype, seed=8)
    ref = FusedSwiGLU.apply(tx, twg, twu)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        outs = [FusedSwiGLU.apply(tx, twg, twu) for _ in range(4)]
    s.synchronize()
    for o in outs:
        assert torch.equal(o, ref)


def test_result_leading_dimension_beyond_the_tiled_kernels_limit(oracle):
    """The tiled kernels address the rows of a wave's results through 32-bit byte offsets, so results whose leading
    dimension reaches 2^23 elements take the edge kernel (selection code 0) and come out the same."""
    dtype, T, D, I = torch.bfloat16, 4, 64, 64
    ldo = 1 << 23
    L = _abi.lib()
    assert L.fsw_uses_tiled_kernel(0, 256, D, I, D, I, ldo - 8, I, 16) == 1
    assert L.fsw_uses_tiled_kernel(0, 256, D, I, D, I, ldo, I, 16) == 0
    (x, wg, wu, _), (tx, twg, twu, _) = make(oracle, (1, T, D, I), dtype, seed=5)
    tx = tx[0].contiguous()
    big = [torch.zeros(T * ldo, device=DEV, dtype=dtype) for _ in range(3)]
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(L.fsw_swiglu_forward(tx.data_ptr(), twg.data_ptr(), twu.data_ptr(), *(b.data_ptr() for b in big),
                                    T, D, I, D, I, ldo, _abi.DTYPE_BF16, stream))
    torch.cuda.synchronize()
    want = oracle.fused_swiglu_fwd(x[0], wg, wu)
    for b, w in zip(big, want):
        got = b.view(T, ldo)[:, :I]
        assert oracle.rel_error(np64(got), w) < 1e-2
        assert not b.view(T, ldo)[:, I:I + 64].any()      # nothing beyond the rows


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["DI", "ID"])
@pytest.mark.parametrize("shape", [(2, 136, 264, 520), (1, 2048, 256, 768), (3, 50, 72, 65), (1, 4096, 2048, 1024)],
                         ids=lambda s: "x".join(map(str, s)))
def test_backward_in_one_call_equals_the_three_steps(oracle, dtype, out_in, shape):
    """fsw_swiglu_backward (fused_swiglu/swiglu.py:34-58 as one library call) enqueues the same three kernels as
    elementwise_backward + fused_input_grad + fused_weight_grad: identical bits, against the oracle, and with
    either gradient switched off."""
    from fusedswiglu_amd.kernels import _launch
    (x, wg, wu, dy), (tx, twg, twu, tdy) = make(oracle, shape, dtype, seed=31)
    if out_in:
        twg, twu = twg.t().contiguous(), twu.t().contiguous()
    _, tg, tu = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, weights_out_in=out_in)
    dU, dG = _launch.elementwise_backward(tdy, tg, tu, dtype)
    dx3 = _launch.fused_input_grad(dG, dU, twg, twu, dtype, weights_out_in=out_in)
    dwu3, dwg3 = _launch.fused_weight_grad(tx, dU, dG, dtype, weights_out_in=out_in)
    dx1, dwg1, dwu1 = _launch.swiglu_backward(tdy, tx, twg, twu, tg, tu, dtype, weights_out_in=out_in)
    torch.cuda.synchronize()
    assert dx1.shape == tx.shape and dwg1.shape == twg.shape and dwu1.shape == twu.shape
    assert torch.equal(dx1, dx3) and torch.equal(dwg1, dwg3) and torch.equal(dwu1, dwu3)
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dy)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(dx1), o_dx) < tol
    assert oracle.rel_error(np64(dwg1.t() if out_in else dwg1), o_dwg) < tol
    assert oracle.rel_error(np64(dwu1.t() if out_in else dwu1), o_dwu) < tol
    only_x = _launch.swiglu_backward(tdy, tx, twg, twu, tg, tu, dtype, need_weight_grad=False, weights_out_in=out_in)
    only_w = _launch.swiglu_backward(tdy, tx, twg, twu, tg, tu, dtype, need_input_grad=False, weights_out_in=out_in)
    torch.cuda.synchronize()
    assert only_x[1] is None and only_x[2] is None and torch.equal(only_x[0], dx3)
    assert only_w[0] is None and torch.equal(only_w[1], dwg3) and torch.equal(only_w[2], dwu3)
