"""GPU parity at the sizes the benchmark quotes for the nn.Linear weight layout and the few-token down projection,
and for the tiled kernels' tail split (a last, partial round of tiles shared by several workgroups).  Same oracle,
metric and bounds as the other parity tests (rel-L2 <= 1e-2 for bfloat16, fused_swiglu/test_swiglu.py:20, :43-44;
<= 5e-3 for float16), all through the C ABI.  The arrays are too large for a whole-array oracle, so each result is
checked on slices the oracle computes exactly from the matching slices of the inputs: whole token rows of
out / dx / y, whole columns (rows, in the nn.Linear layout) of the weight gradients."""
import numpy as np
import pytest
import torch

from fusedswiglu_amd import _abi, ops
from fusedswiglu_amd.kernels import _launch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.bfloat16: 1e-2, torch.float16: 5e-3}


def np64(t):
    return t.detach().float().cpu().double().numpy()


def randn(shape, dtype, g, scale=1.0):
    return (torch.randn(*shape, device=DEV, dtype=torch.float32, generator=g) * scale).to(dtype)


def check_swiglu_slices(oracle, dtype, out_in, tx, twg, twu, tdy, out, dx, dwg, dwu, rows, cols):
    """out / dx on token rows `rows`, weight gradients on intermediate columns `cols`; weights and their gradients
    are [I, D] when out_in."""
    tol = TOL[dtype]
    r_t, c_t = torch.as_tensor(rows, device=DEV), torch.as_tensor(cols, device=DEV)
    wg64, wu64 = (np64(twg).T, np64(twu).T) if out_in else (np64(twg), np64(twu))   # [D, I]
    xr = np64(tx[r_t])
    errs = {"out": oracle.rel_error(np64(out[r_t]), oracle.fused_swiglu_fwd(xr, wg64, wu64)[0])}
    if dx is not None:
        errs["dx"] = oracle.rel_error(np64(dx[r_t]), oracle.swiglu_backward(xr, wg64, wu64, np64(tdy[r_t]))[0])
        _, o_dwg, o_dwu = oracle.swiglu_backward(np64(tx), wg64[:, cols], wu64[:, cols], np64(tdy[:, c_t]))
        got_g, got_u = (np64(dwg[c_t]).T, np64(dwu[c_t]).T) if out_in else (np64(dwg[:, c_t]), np64(dwu[:, c_t]))
        errs["dWg"], errs["dWu"] = oracle.rel_error(got_g, o_dwg), oracle.rel_error(got_u, o_dwu)
        assert oracle.rel_error(got_g, o_dwu) > 0.1   # gate / up not swapped
    for k, v in errs.items():
        assert np.isfinite(v) and v < tol, f"{k}: rel-L2 {v:.3e} >= {tol}"


def run_swiglu(dtype, out_in, tx, twg, twu, tdy):
    tx, twg, twu = (t.detach().clone().requires_grad_(True) for t in (tx, twg, twu))
    out = ops.swiglu(tx, twg, twu, autocast_dtype=None, weights_out_in=out_in)
    out.backward(tdy)
    torch.cuda.synchronize()
    return out.detach(), tx.grad, twg.grad, twu.grad


def test_linear_layout_headline_shape_forward_backward(oracle):
    """8192 tokens, d = 4096 -> 12288 with [I, D] weights: the three tiled kernels of that layout at the size
    the benchmark times them."""
    dtype, T, D, I = torch.bfloat16, 8192, 4096, 12288
    g = torch.Generator(device=DEV).manual_seed(11)
    tx, tdy = randn((T, D), dtype, g), randn((T, I), dtype, g)
    twg, twu = randn((I, D), dtype, g, D ** -0.5), randn((I, D), dtype, g, D ** -0.5)
    assert _abi.lib().fsw_uses_tiled_kernel(_abi.WEIGHTS_OUT_IN, T, D, I, D, D, I, I, 16) == 1
    out, dx, dwg, dwu = run_swiglu(dtype, True, tx, twg, twu, tdy)
    assert dwg.shape == (I, D)
    check_swiglu_slices(oracle, dtype, True, tx, twg, twu, tdy, out, dx, dwg, dwu,
                        rows=[0, 255, 256, 4097, 8191], cols=[0, 127, 128, 6145, 12287])


@pytest.mark.parametrize("M", [16, 64, 128, 256])
def test_linear_layout_few_token_forward_full_width(oracle, M):
    """x [M, 8192], W [28672, 8192]: the weight-streaming forward of the nn.Linear layout (the tiled kernel with a
    single row of tiles above 128 tokens) at the size the benchmark times it."""
    dtype, D, I = torch.bfloat16, 8192, 28672
    g = torch.Generator(device=DEV).manual_seed(100 + M)
    tx = randn((M, D), dtype, g)
    twg, twu = randn((I, D), dtype, g, D ** -0.5), randn((I, D), dtype, g, D ** -0.5)
    assert _abi.lib().fsw_uses_tiled_kernel(_abi.WEIGHTS_OUT_IN, M, D, I, D, D, I, I, 16) == (2 if M <= 128 else 1)
    with torch.no_grad():
        out = ops.swiglu(tx, twg, twu, autocast_dtype=None, weights_out_in=True)
    torch.cuda.synchronize()
    rows = sorted({0, M - 1, M // 2, M // 3, (2 * M) // 3, 7 % M})
    check_swiglu_slices(oracle, dtype, True, tx, twg, twu, None, out, None, None, None, rows=rows, cols=[0])
    # every column block in its place: per-column error on those rows
    want = oracle.fused_swiglu_fwd(np64(tx[rows]), np64(twg).T, np64(twu).T)[0]
    col_err = np.linalg.norm(np64(out[rows]) - want, axis=0) / (np.linalg.norm(want, axis=0) + 1e-30)
    assert col_err.max() < 0.2


@pytest.mark.parametrize("out_in", [False, True], ids=["w_down_IxD", "w_down_DxI"])
@pytest.mark.parametrize("T", [16, 64, 128])
def test_few_token_down_projection_full_size(oracle, T, out_in):
    """y [T, 8192] = act [T, 28672] W_down and its input gradient in both storage orders of W_down: the streaming
    kernel with the reduction split over the workgroups, at the size the benchmark times it."""
    dtype, I, D = torch.bfloat16, 28672, 8192
    g = torch.Generator(device=DEV).manual_seed(200 + T)
    tact, tdy = randn((T, I), dtype, g), randn((T, D), dtype, g)
    twd = randn((D, I) if out_in else (I, D), dtype, g, I ** -0.5)
    y = _launch.down_proj_forward(tact, twd, dtype, weights_out_in=out_in)
    d_act = _launch.down_proj_input_grad(tdy, twd, dtype, weights_out_in=out_in)
    torch.cuda.synchronize()
    assert y.shape == (T, D) and d_act.shape == (T, I)
    tol = TOL[dtype]
    rng = np.random.default_rng(T)
    dcols = np.unique(np.concatenate([[0, D - 1, 4095, 4096], rng.integers(0, D, 60)]))   # columns of y
    icols = np.unique(np.concatenate([[0, I - 1, 14335, 14336], rng.integers(0, I, 60)]))  # columns of d_act
    dc, ic = torch.as_tensor(dcols, device=DEV), torch.as_tensor(icols, device=DEV)
    wd_d = np64(twd[dc]).T if out_in else np64(twd[:, dc])      # [I, |dcols|]
    wd_i = np64(twd[:, ic]).T if out_in else np64(twd[ic])      # [|icols|, D]
    assert oracle.rel_error(np64(y[:, dc]), oracle.down_proj_fwd(np64(tact), wd_d)) < tol
    assert oracle.rel_error(np64(d_act[:, ic]), oracle.down_proj_backward(np64(tact[:, ic]), wd_i, np64(tdy))[0]) < tol


# dx has 17 x 16 = 272 tiles at (4352, 4096, 2048) and the weight gradients 8 x 34 = 272 at (4096, 2048, 4352):
# one full round of 256 workgroups and a tail of 16 tiles, each split over four workgroups; the ragged shape
# has edge tiles in the tail as well.  C3 (fp16, I = 11008: 1376 weight-gradient tiles, a tail of 96 split in
# two) runs in the full-size tests.
TAIL_SHAPES = [(4352, 4096, 2048), (4096, 2048, 4352), (4296, 4104, 2120)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["DI", "ID"])
@pytest.mark.parametrize("tdi", TAIL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_tail_split_of_the_gradient_gemms(oracle, dtype, out_in, tdi):
    """Gradient GEMMs whose tiles leave a short last round: rows and columns through every tile, so every tile of
    the tail (they are scattered over the result by the XCD-aware tile order) is compared with the oracle."""
    T, D, I = tdi
    L = _abi.lib()
    flag = _abi.WEIGHTS_OUT_IN if out_in else 0
    assert L.fsw_workspace_bytes(1 | flag, T, D, I) > 0 or L.fsw_workspace_bytes(2 | flag, T, D, I) > 0
    g = torch.Generator(device=DEV).manual_seed(T + I)
    tx, tdy = randn((T, D), dtype, g), randn((T, I), dtype, g, 0.1)
    wshape = (I, D) if out_in else (D, I)
    twg, twu = randn(wshape, dtype, g, D ** -0.5), randn(wshape, dtype, g, D ** -0.5)
    out, dx, dwg, dwu = run_swiglu(dtype, out_in, tx, twg, twu, tdy)
    rows = np.unique(np.concatenate([np.arange(5, T, 64), [0, T - 1]]))     # every 256-row and 128-row tile
    cols = np.unique(np.concatenate([np.arange(3, I, 64), [0, I - 1]]))     # every 128-column tile
    check_swiglu_slices(oracle, dtype, out_in, tx, twg, twu, tdy, out, dx, dwg, dwu, rows=rows, cols=cols)
    # dx on columns through every tile as well (its tail tiles are tiles of [T, D])
    out2, dx2, dwg2, dwu2 = run_swiglu(dtype, out_in, tx, twg, twu, tdy)
    assert torch.equal(dx, dx2) and torch.equal(dwg, dwg2) and torch.equal(dwu, dwu2)   # fixed summation order


# Shapes that take each form of the tiled kernels (eight waves for short reductions, four waves for long ones),
# with and without edge tiles, a split reduction and a tail split.
WHOLE_ARRAY_SHAPES = [(4096, 2048, 4352), (2048, 4096, 2048), (512, 2048, 512), (4360, 2056, 4232), (1000, 1032, 776),
                      (8192, 4096, 5504)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["DI", "ID"])
@pytest.mark.parametrize("tdi", WHOLE_ARRAY_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_every_element_of_every_result(oracle, dtype, out_in, tdi):
    """The oracle checks above compare slices; a fault confined to a few rows or lanes of a tile could sit between
    them.  Here every element of out, g, u, dx, dWg and dWu is compared on the GPU with fp32 products of the same
    16-bit inputs (element-wise bound: a few roundings of the result's magnitude, far below any stale or unconverted
    value), the oracle confirms the fp32 products on a slice, and a second run must reproduce every bit."""
    T, D, I = tdi
    g = torch.Generator(device=DEV).manual_seed(7 * T + I)
    tx, tdy = randn((T, D), dtype, g), randn((T, I), dtype, g)
    wshape = (I, D) if out_in else (D, I)
    twg, twu = randn(wshape, dtype, g, D ** -0.5), randn(wshape, dtype, g, D ** -0.5)
    def run():
        out, pg, pu = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, weights_out_in=out_in)
        dU, dG = _launch.elementwise_backward(tdy, pg, pu, dtype)
        dx = _launch.fused_input_grad(dG, dU, twg, twu, dtype, weights_out_in=out_in)
        dwu, dwg = _launch.fused_weight_grad(tx, dU, dG, dtype, weights_out_in=out_in)
        # the gating gradient again, from x and the weights (forward kernel with the gating-gradient epilogue)
        rU, rG = _launch.gating_grad_recompute(tdy, tx, twg, twu, dtype, weights_out_in=out_in)
        torch.cuda.synchronize()
        return out, pg, pu, dG, dU, dx, dwg, dwu, rU, rG

    out, pg, pu, dG, dU, dx, dwg, dwu, rU, rG = run()
    xf, dyf = tx.float(), tdy.float()
    wgf, wuf = (twg.float().t(), twu.float().t()) if out_in else (twg.float(), twu.float())   # [D, I]
    rg, ru = xf @ wgf, xf @ wuf
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11

    def close(name, got, want, scale):
        err = (got.float() - want).abs()
        bound = 4 * eps * want.abs() + scale
        bad = int((~(err <= bound)).sum())   # NaN counts as bad
        assert bad == 0, f"{name}: {bad} elements outside the bound, worst {err.max().item():.3e}"

    k_fwd, k_dx, k_dw = D ** 0.5, (2 * I) ** 0.5, T ** 0.5
    close("g", pg, rg, 1e-5 * k_fwd)
    close("u", pu, ru, 1e-5 * k_fwd)
    close("out", out, torch.nn.functional.silu(rg) * ru, 1e-5 * k_fwd)
    sg = torch.sigmoid(rg)
    close("recomputed dU", rU, dyf * rg * sg, 1e-5 * k_fwd)
    close("recomputed dG", rG, dyf * ru * (sg + rg * sg * (1 - sg)), 4e-5 * k_fwd)
    # the gradients from the kernels' own (rounded) dG, dU, so that only the GEMM under test contributes
    dGf, dUf = dG.float(), dU.float()
    close("dx", dx, dGf @ wgf.t() + dUf @ wuf.t(), 2e-5 * k_dx * dGf.abs().max().item())
    rdwg, rdwu = xf.t() @ dGf, xf.t() @ dUf
    if out_in:
        rdwg, rdwu = rdwg.t(), rdwu.t()
    close("dWg", dwg, rdwg, 2e-5 * k_dw * dGf.abs().max().item())
    close("dWu", dwu, rdwu, 2e-5 * k_dw * dUf.abs().max().item())
    # the fp32 products themselves against the oracle on a few token rows
    rows = [0, T // 3, T - 1]
    wg64, wu64 = np64(wgf), np64(wuf)
    want = oracle.fused_swiglu_fwd(np64(tx[rows]), wg64, wu64)[0]
    assert oracle.rel_error(np64((torch.nn.functional.silu(rg) * ru)[rows]), want) < 1e-5
    again = run()
    for a, b in zip((out, pg, pu, dG, dU, dx, dwg, dwu, rU, rG), again):
        assert torch.equal(a, b)


FEW_TOKEN_WHOLE = [(16, 8192, 28672), (64, 4096, 12288), (128, 8192, 28672), (100, 1032, 7176), (256, 8192, 28672),
                   (200, 4096, 11008)]


@pytest.mark.parametrize("out_in", [False, True], ids=["DI", "ID"])
@pytest.mark.parametrize("tdi", FEW_TOKEN_WHOLE, ids=lambda s: "x".join(map(str, s)))
def test_every_element_of_the_few_token_forward_and_down_projection(oracle, out_in, tdi):
    """The weight-streaming kernels (and the tiled kernel with a single row of tiles above 128 tokens) at full
    width: every element of out, of the down projection y = out W_down and of its input gradient against fp32
    products of the same inputs on the GPU, the fp32 products against the oracle on one row, and a second run bit
    for bit."""
    T, D, I = tdi
    dtype = torch.bfloat16
    g = torch.Generator(device=DEV).manual_seed(3 * T + D)
    tx = randn((T, D), dtype, g)
    wshape = (I, D) if out_in else (D, I)
    twg, twu = randn(wshape, dtype, g, D ** -0.5), randn(wshape, dtype, g, D ** -0.5)
    twd = randn((D, I) if out_in else (I, D), dtype, g, I ** -0.5)
    tdy = randn((T, D), dtype, g)

    def run():
        with torch.no_grad():
            out = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, save_preactivations=False, weights_out_in=out_in)[0]
            y = _launch.down_proj_forward(out, twd, dtype, weights_out_in=out_in)
            d_act = _launch.down_proj_input_grad(tdy, twd, dtype, weights_out_in=out_in)
        torch.cuda.synchronize()
        return out, y, d_act

    out, y, d_act = run()
    wgf, wuf = (twg.float().t(), twu.float().t()) if out_in else (twg.float(), twu.float())      # [D, I]
    wdf = twd.float().t() if out_in else twd.float()                                              # [I, D]
    xf = tx.float()
    want = torch.nn.functional.silu(xf @ wgf) * (xf @ wuf)
    eps = 2.0 ** -8

    def close(name, got, ref, scale):
        err = (got.float() - ref).abs()
        bad = int((~(err <= 4 * eps * ref.abs() + scale)).sum())
        assert bad == 0, f"{name}: {bad} elements outside the bound, worst {err.max().item():.3e}"

    close("out", out, want, 1e-5 * D ** 0.5)
    close("y", y, out.float() @ wdf, 2e-5 * I ** 0.5 * out.float().abs().max().item())
    close("d_act", d_act, tdy.float() @ wdf.t(), 2e-5 * D ** 0.5 * tdy.float().abs().max().item())
    row = [T // 2]
    o_row = oracle.fused_swiglu_fwd(np64(tx[row]), np64(wgf), np64(wuf))[0]
    assert oracle.rel_error(np64(want[row]), o_row) < 1e-5
    for a, b in zip((out, y, d_act), run()):
        assert torch.equal(a, b)
