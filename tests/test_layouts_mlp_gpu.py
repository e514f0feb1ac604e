"""GPU parity of what sits either side of the reference's path in real model code: weights kept in
nn.Linear's [d_intermediate, d_model] layout (read in place by their own tiled-kernel variants) and the down
projection that follows the SwiGLU.  Same oracle, metric and bounds as the parity tests of the path itself
(rel-L2 <= 1e-2 for bfloat16, fused_swiglu/test_swiglu.py:20; <= 5e-3 for float16), all through the C ABI."""
import numpy as np
import pytest
import torch

import fusedswiglu_amd as fsw
from fusedswiglu_amd import _abi, ops
from fusedswiglu_amd.kernels import _launch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.bfloat16: 1e-2, torch.float16: 5e-3}
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}
SHAPES = [
    (2, 256, 256, 512),    # full tiles
    (1, 520, 264, 392),    # multiples of 8 only: edge tiles in every dimension
    (3, 100, 1032, 776),
    (1, 7, 8, 8),          # tiny
    (2, 33, 72, 65),       # I not a multiple of 8 -> edge-shape kernel
    (1, 257, 100, 130),    # nothing aligned
    (4, 512, 256, 768),    # few output tiles, long reductions: split reductions in every gradient GEMM
    (1, 64, 4096, 1024),   # few tokens: the weight-streaming kernels in either layout, the down projection with a split
]


def np64(t):
    return t.detach().float().cpu().double().numpy()


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def make(oracle, shape, dtype, seed):
    B, S, D, I = shape
    x, wg, wu, dact = oracle.make_input_weights(B, S, D, I, seed=seed, dtype=NAME[dtype], dout_scale=0.1)
    rng = np.random.default_rng(seed + 1000)
    rnd = oracle.rounder(NAME[dtype])
    wd = rnd(rng.standard_normal((I, D)) / I ** 0.5)
    dy = rnd(0.1 * rng.standard_normal((B, S, D)))
    return x, wg, wu, wd, dact, dy


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_layout_weights_forward_backward(oracle, dtype, shape):
    """swiglu(..., weights_out_in=True) on [I, D] weights against the oracle evaluated on their transposes;
    the weight gradients come back in [I, D] too."""
    x, wg, wu, _, dact, _ = make(oracle, shape, dtype, seed=3)
    tx = dev(x, dtype).requires_grad_(True)
    twg = dev(wg.T, dtype).requires_grad_(True)   # [I, D], contiguous: nn.Linear(d_model, d_int).weight
    twu = dev(wu.T, dtype).requires_grad_(True)
    out = ops.swiglu(tx, twg, twu, autocast_dtype=None, weights_out_in=True)
    out.backward(dev(dact, dtype))
    torch.cuda.synchronize()
    o_out = oracle.fused_swiglu_fwd(x, wg, wu)[0]
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dact)
    tol = TOL[dtype]
    assert twg.grad.shape == twg.shape and twu.grad.shape == twu.shape
    assert oracle.rel_error(np64(out), o_out) < tol
    assert oracle.rel_error(np64(tx.grad), o_dx) < tol
    assert oracle.rel_error(np64(twg.grad), o_dwg.T) < tol and oracle.rel_error(np64(twu.grad), o_dwu.T) < tol
    assert oracle.rel_error(np64(twg.grad), o_dwu.T) > 0.1  # gate/up not swapped


@pytest.mark.parametrize("shape", [(2, 136, 264, 520), (1, 300, 256, 384), (3, 50, 72, 65)], ids=lambda s: "x".join(map(str, s)))
def test_both_layouts_agree_and_recompute_works_in_linear_layout(oracle, shape):
    """The two weight layouts are the same arithmetic in a different tile order: results agree to well inside
    the bound; the memory-saving backward and the packed [2I, D] weight work in the nn.Linear layout as well."""
    dtype = torch.bfloat16
    x, wg, wu, _, dact, _ = make(oracle, shape, dtype, seed=5)
    I = shape[3]
    res = {}
    for oi in (False, True):
        for mode in ("plain", "recompute", "packed"):
            tx = dev(x, dtype).requires_grad_(True)
            a, b = (dev(wg.T, dtype), dev(wu.T, dtype)) if oi else (dev(wg, dtype), dev(wu, dtype))
            if mode == "packed":
                w = torch.cat([a, b], dim=0 if oi else 1).contiguous().requires_grad_(True)
                out = ops.swiglu_packed(tx, w, autocast_dtype=None, weights_out_in=oi)
                out.backward(dev(dact, dtype))
                gw = w.grad
                dwg, dwu = (gw[:I], gw[I:]) if oi else (gw[:, :I], gw[:, I:])
            else:
                a.requires_grad_(True), b.requires_grad_(True)
                out = ops.swiglu(tx, a, b, autocast_dtype=None, recompute=(mode == "recompute"), weights_out_in=oi)
                out.backward(dev(dact, dtype))
                dwg, dwu = a.grad, b.grad
            res[(oi, mode)] = (np64(out), np64(tx.grad), np64(dwg.t() if oi else dwg), np64(dwu.t() if oi else dwu))
    torch.cuda.synchronize()
    exact = (oracle.fused_swiglu_fwd(x, wg, wu)[0],) + oracle.swiglu_backward(x, wg, wu, dact)
    for key, got in res.items():
        for g, e in zip(got, exact):
            assert oracle.rel_error(g, e) < TOL[dtype], key
    for mode in ("plain", "recompute", "packed"):
        for g0, g1 in zip(res[(False, mode)], res[(True, mode)]):
            assert oracle.rel_error(g1, g0) < 4e-3, mode


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["w_down_IxD", "w_down_DxI"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_down_projection_launchers(oracle, dtype, out_in, shape):
    """fsw_down_proj_forward / _input_grad / _weight_grad against the oracle, for both layouts of W_down."""
    x, wg, wu, wd, _, dy = make(oracle, shape, dtype, seed=7)
    act = oracle.rounder(NAME[dtype])(oracle.fused_swiglu_fwd(x, wg, wu)[0])
    tact, tdy = dev(act, dtype), dev(dy, dtype)
    twd = dev(wd.T if out_in else wd, dtype)
    y = _launch.down_proj_forward(tact, twd, dtype, weights_out_in=out_in)
    d_act = _launch.down_proj_input_grad(tdy, twd, dtype, weights_out_in=out_in)
    d_w = _launch.down_proj_weight_grad(tact, tdy, dtype, weights_out_in=out_in)
    torch.cuda.synchronize()
    o_da, o_dw = oracle.down_proj_backward(act, wd, dy)
    tol = TOL[dtype]
    assert y.shape == tuple(shape[:2]) + (shape[2],) and d_act.shape == tact.shape and d_w.shape == twd.shape
    assert oracle.rel_error(np64(y), oracle.down_proj_fwd(act, wd)) < tol
    assert oracle.rel_error(np64(d_act), o_da) < tol
    assert oracle.rel_error(np64(d_w), o_dw.T if out_in else o_dw) < tol


# (T, I, D); the last three have I a multiple of 128, so that the input gradient streams W_down as well (half of
# its I result columns must be a multiple of 64, or of 8 for [I, D] storage), with and without a split reduction
FEW_TOKENS_DOWN = [(1, 72, 128), (16, 520, 256), (33, 1096, 384), (64, 4104, 512), (100, 8200, 1024), (128, 2056, 1152),
                   (16, 1024, 4096), (64, 28672, 1024), (128, 256, 8192)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["w_down_IxD", "w_down_DxI"])
@pytest.mark.parametrize("tid", FEW_TOKENS_DOWN, ids=lambda s: "x".join(map(str, s)))
def test_few_token_down_projection(oracle, dtype, out_in, tid):
    """Up to 128 tokens the down projection streams the weights on the kernel of the few-token forward, as a plain
    GEMM over the two column halves of W_down with the reduction split into the caller's scratch; so does its
    input gradient when half of I is aligned (selection code 2, else the tiled kernel, code 1): against the oracle
    with scratch (the launcher asks the library for it), and through the raw ABI without scratch (no split), which
    must agree to within the rounding of one more fp32 summation order."""
    T, I, D = tid
    flag = _abi.WEIGHTS_OUT_IN if out_in else 0
    uses = _abi.lib().fsw_uses_tiled_kernel
    ldw = I if out_in else D
    assert uses(4 | flag, T, D, I, D, ldw, I, ldw, 16) == 2      # D / 2 is a multiple of 64 in every case
    half_ok = (I // 2) % (64 if out_in else 8) == 0 and I % 2 == 0
    assert uses(5 | flag, T, D, I, D, ldw, I, ldw, 16) == (2 if half_ok else 1)
    assert uses(6 | flag, T, D, I, D, ldw, I, ldw, 16) == 1
    rng = np.random.default_rng(T + I)
    rnd = oracle.rounder(NAME[dtype])
    act = rnd(rng.standard_normal((T, I)))
    wd = rnd(rng.standard_normal((I, D)) / I ** 0.5)
    dy = rnd(rng.standard_normal((T, D)))
    tact, tdy, twd = dev(act, dtype), dev(dy, dtype), dev(wd.T if out_in else wd, dtype)
    y = _launch.down_proj_forward(tact, twd, dtype, weights_out_in=out_in)
    d_act = _launch.down_proj_input_grad(tdy, twd, dtype, weights_out_in=out_in)
    y_nosplit = torch.empty_like(y)
    L, p = _abi.lib(), lambda t: t.data_ptr()
    code = (_abi.DTYPE_BF16 if dtype == torch.bfloat16 else _abi.DTYPE_FP16) | (_abi.WEIGHTS_OUT_IN if out_in else 0)
    _abi.check(L.fsw_down_proj_forward(p(tact), p(twd), p(y_nosplit), T, I, D, I, twd.shape[1], D, None, 0, code,
                                       torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    o_da, _ = oracle.down_proj_backward(act, wd, dy)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(y), oracle.down_proj_fwd(act, wd)) < tol
    assert oracle.rel_error(np64(y_nosplit), oracle.down_proj_fwd(act, wd)) < tol
    assert oracle.rel_error(np64(y), np64(y_nosplit)) < tol / 2
    assert oracle.rel_error(np64(d_act), o_da) < tol


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("keep_layout", [True, False], ids=["linear_layout", "reference_layout"])
def test_mlp_module_from_linear(oracle, dtype, keep_layout):
    """SwiGLUMLP built from three nn.Linear projections (a Llama-style MLP): forward and all four gradients
    against the oracle's composition; with keep_layout the module computes on the projections' own weights."""
    shape = (2, 136, 264, 520)
    B, S, D, I = shape
    x, wg, wu, wd, _, dy = make(oracle, shape, dtype, seed=9)
    gate = torch.nn.Linear(D, I, bias=False, device=DEV, dtype=dtype)
    up = torch.nn.Linear(D, I, bias=False, device=DEV, dtype=dtype)
    down = torch.nn.Linear(I, D, bias=False, device=DEV, dtype=dtype)
    with torch.no_grad():
        gate.weight.copy_(dev(wg.T, dtype)), up.weight.copy_(dev(wu.T, dtype)), down.weight.copy_(dev(wd.T, dtype))
    m = fsw.SwiGLUMLP.from_linear(gate, up, down, keep_layout=keep_layout)
    if keep_layout:
        assert m.w_down is down.weight and m.swiglu.w_gate is gate.weight
    tx = dev(x, dtype).requires_grad_(True)
    y = m(tx)
    y.backward(dev(dy, dtype))
    torch.cuda.synchronize()
    o_y, o_dx, o_dwg, o_dwu, o_dwd = oracle.mlp_fwd_bwd(x, wg, wu, wd, dy)
    tol = TOL[dtype]
    tr = (lambda a: a.T) if keep_layout else (lambda a: a)
    assert oracle.rel_error(np64(y), o_y) < tol
    assert oracle.rel_error(np64(tx.grad), o_dx) < tol
    assert oracle.rel_error(np64(m.swiglu.w_gate.grad), tr(o_dwg)) < tol
    assert oracle.rel_error(np64(m.swiglu.w_up.grad), tr(o_dwu)) < tol
    assert oracle.rel_error(np64(m.w_down.grad), tr(o_dwd)) < tol
    # the eager PyTorch MLP on the same modules agrees too (a second, independent check of the layouts)
    ref = down(torch.nn.functional.silu(gate(tx.detach())) * up(tx.detach()))
    assert oracle.rel_error(np64(y), np64(ref)) < 2 * tol


FEW_TOKENS = [(1, 8, 8), (7, 72, 136), (16, 520, 392), (33, 1032, 136), (64, 200, 1160), (65, 64, 264), (128, 1096, 520),
              (129, 264, 520), (256, 520, 392)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("out_in", [False, True], ids=["DI", "ID"])
@pytest.mark.parametrize("tdi", FEW_TOKENS, ids=lambda s: "x".join(map(str, s)))
def test_few_token_forward_in_both_layouts(oracle, dtype, out_in, tdi):
    """Up to 128 tokens the forward runs on the weight-streaming kernels (selection code 2), one per weight
    layout; up to 256 the tiled kernel has a single row of tiles and streams the weights past the caches: out and
    the saved pre-activations against the oracle, with reductions that are not multiples of a stage (64
    elements), ragged last column blocks and row counts on both sides of every variant."""
    T, D, I = tdi
    x, wg, wu, _, _, _ = make(oracle, (1, T, D, I), dtype, seed=T + D)
    tx = dev(x[0], dtype)
    twg, twu = (dev(wg.T, dtype), dev(wu.T, dtype)) if out_in else (dev(wg, dtype), dev(wu, dtype))
    ldw = D if out_in else I
    flag = _abi.WEIGHTS_OUT_IN if out_in else 0
    assert _abi.lib().fsw_uses_tiled_kernel(flag, T, D, I, D, ldw, I, I, 16) == (2 if T <= 128 else 1)
    out, g, u = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, weights_out_in=out_in)
    out_only = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, save_preactivations=False, weights_out_in=out_in)[0]
    torch.cuda.synchronize()
    o_out, o_g, o_u = oracle.fused_swiglu_fwd(x[0], wg, wu)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(out), o_out) < tol
    assert oracle.rel_error(np64(g), o_g) < tol and oracle.rel_error(np64(u), o_u) < tol
    assert torch.equal(out, out_only)


@pytest.mark.parametrize("seed", range(16))
def test_few_token_random_shapes(oracle, seed):
    """Seeded random few-token problems (T <= 128, dimensions multiples of 8 so that the streaming kernels run):
    SwiGLU forward in a random layout and element type, then the down projection in a random storage order,
    each against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    dtype = (torch.bfloat16, torch.float16)[seed & 1]
    T = int(rng.integers(1, 129))
    D = 8 * int(rng.integers(1, 160))
    I = 16 * int(rng.integers(1, 200))       # the down projection needs I / 2 aligned as well
    out_in, down_out_in = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    rnd = oracle.rounder(NAME[dtype])
    x = rnd(rng.standard_normal((T, D)))
    wg, wu = rnd(rng.standard_normal((D, I)) / D ** 0.5), rnd(rng.standard_normal((D, I)) / D ** 0.5)
    wd = rnd(rng.standard_normal((I, D)) / I ** 0.5)
    tx = dev(x, dtype)
    twg, twu = (dev(wg.T, dtype), dev(wu.T, dtype)) if out_in else (dev(wg, dtype), dev(wu, dtype))
    out, g, u = _launch.fused_swiglu_fwd(tx, twg, twu, dtype, weights_out_in=out_in)
    torch.cuda.synchronize()
    o_out, o_g, o_u = oracle.fused_swiglu_fwd(x, wg, wu)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(out), o_out) < tol, (T, D, I, out_in)
    assert oracle.rel_error(np64(g), o_g) < tol and oracle.rel_error(np64(u), o_u) < tol
    act = np64(out)
    y = _launch.down_proj_forward(out, dev(wd.T if down_out_in else wd, dtype), dtype, weights_out_in=down_out_in)
    torch.cuda.synchronize()
    assert oracle.rel_error(np64(y), oracle.down_proj_fwd(act, wd)) < tol, (T, D, I, down_out_in)


def test_linear_layout_full_size_forward_slices(oracle):
    """The headline shape with nn.Linear-layout weights: whole token rows of out against the oracle."""
    dtype, T, D, I = torch.bfloat16, 8192, 4096, 12288
    g = torch.Generator(device=DEV).manual_seed(0)
    tx = torch.randn(T, D, device=DEV, dtype=torch.float32, generator=g).to(dtype)
    twg = (torch.randn(I, D, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    twu = (torch.randn(I, D, device=DEV, dtype=torch.float32, generator=g) / D ** 0.5).to(dtype)
    assert _abi.lib().fsw_uses_tiled_kernel(_abi.WEIGHTS_OUT_IN, T, D, I, D, D, I, I, 16) == 1
    with torch.no_grad():
        out = ops.swiglu(tx, twg, twu, autocast_dtype=None, weights_out_in=True)
    rows = torch.tensor([0, 1, 4097, 8191], device=DEV)
    want = oracle.fused_swiglu_fwd(np64(tx[rows]), np64(twg).T, np64(twu).T)[0]
    assert oracle.rel_error(np64(out[rows]), want) < TOL[dtype]


def test_new_operators_pass_opcheck(oracle):
    """Schema, fake implementation and autograd registration of the layout-flagged and down-projection operators."""
    dtype, shape = torch.bfloat16, (2, 16, 32, 48)
    x, wg, wu, wd, dact, dy = make(oracle, shape, dtype, seed=13)
    tx, tact, tdy = dev(x, dtype), dev(dact, dtype), dev(dy, dtype)
    tests = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_dynamic")
    for oi in (False, True):
        twg, twu = (dev(wg.T, dtype), dev(wu.T, dtype)) if oi else (dev(wg, dtype), dev(wu, dtype))
        twd = dev(wd.T if oi else wd, dtype)
        torch.library.opcheck(ops.swiglu_forward, (tx.clone().requires_grad_(True), twg, twu.clone().requires_grad_(True), True, oi),
                              test_utils=tests)
        torch.library.opcheck(ops.down_proj_forward, (tact.clone().requires_grad_(True), twd.clone().requires_grad_(True), oi),
                              test_utils=tests)
        torch.library.opcheck(ops.down_proj_backward, (tdy, tact, twd, True, True, oi), test_utils=tests[:3])
    # the functional block end to end, fp16 through autocast from fp32 inputs
    with torch.autocast("cuda", dtype=torch.float16):
        y = ops.swiglu_mlp(tx.float(), dev(wg, dtype).float(), dev(wu, dtype).float(), dev(wd, dtype).float(),
                           autocast_dtype=torch.float16)
    assert y.dtype == torch.float16
    assert oracle.rel_error(np64(y), oracle.mlp_fwd_bwd(x, wg, wu, wd, dy)[0]) < 1e-2
