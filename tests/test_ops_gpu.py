"""GPU tests of the torch.library operators, the packed-weight entry point and the nn.Module wrapper:
same oracle, metric and bounds as the parity tests of the autograd Functions."""
import numpy as np
import pytest
import torch

import fusedswiglu_amd as fsw
from fusedswiglu_amd import ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.bfloat16: 1e-2, torch.float16: 5e-3}  # rel-L2 bounds (bf16: test_swiglu.py:20)
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}


def np64(t):
    return t.detach().float().cpu().double().numpy()


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def inputs(oracle, shape, dtype, seed):
    B, S, D, I = shape
    host = oracle.make_input_weights(B, S, D, I, seed=seed, dtype=NAME[dtype], dout_scale=0.1)
    return host, tuple(dev(a, dtype) for a in host)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("packed", [False, True], ids=["two_weights", "packed"])
def test_module_forward_backward(oracle, dtype, packed):
    shape = (2, 136, 264, 520)
    (x, wg, wu, dy), (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=11)
    m = fsw.SwiGLU(shape[2], shape[3], dtype=dtype, device=DEV, packed=packed)
    with torch.no_grad():
        if packed:
            m.w_gate_up.copy_(torch.cat([twg, twu], dim=1))
        else:
            m.w_gate.copy_(twg)
            m.w_up.copy_(twu)
    tx = tx.clone().requires_grad_(True)
    out = m(tx)
    out.backward(tdy)
    torch.cuda.synchronize()
    o_out = oracle.fused_swiglu_fwd(x, wg, wu)[0]
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dy)
    tol = TOL[dtype]
    assert oracle.rel_error(np64(out), o_out) < tol
    assert oracle.rel_error(np64(tx.grad), o_dx) < tol
    if packed:
        g = m.w_gate_up.grad
        assert g.shape == (shape[2], 2 * shape[3]) and g.is_contiguous()
        dwg, dwu = g[:, :shape[3]], g[:, shape[3]:]
    else:
        dwg, dwu = m.w_gate.grad, m.w_up.grad
    assert oracle.rel_error(np64(dwg), o_dwg) < tol and oracle.rel_error(np64(dwu), o_dwu) < tol
    assert oracle.rel_error(np64(dwg), o_dwu) > 0.1  # halves not swapped
    # inference path: no pre-activations, same values
    with torch.no_grad():
        assert torch.equal(m(tx), out)


def test_packed_and_function_paths_agree_bitwise(oracle):
    """The packed entry point only changes strides: same kernels, same bits as FusedSwiGLU.apply."""
    dtype, shape = torch.bfloat16, (1, 300, 256, 384)
    _, (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=12)
    a = [t.clone().requires_grad_(True) for t in (tx, twg, twu)]
    out_a = fsw.FusedSwiGLU.apply(*a)
    out_a.backward(tdy)
    xb = tx.clone().requires_grad_(True)
    wb = torch.cat([twg, twu], dim=1).requires_grad_(True)
    out_b = fsw.swiglu_packed(xb, wb)
    out_b.backward(tdy)
    xc = [t.clone().requires_grad_(True) for t in (tx, twg, twu)]
    out_c = fsw.swiglu(*xc)
    out_c.backward(tdy)
    torch.cuda.synchronize()
    I = shape[3]
    assert torch.equal(out_a, out_b) and torch.equal(out_a, out_c)
    assert torch.equal(a[0].grad, xb.grad) and torch.equal(a[0].grad, xc[0].grad)
    assert torch.equal(a[1].grad, wb.grad[:, :I]) and torch.equal(a[2].grad, wb.grad[:, I:])
    assert torch.equal(a[1].grad, xc[1].grad) and torch.equal(a[2].grad, xc[2].grad)


def test_operator_registration_passes_opcheck(oracle):
    """Schema, fake implementation, autograd registration and AOT dispatch of both operators."""
    dtype = torch.bfloat16
    _, (tx, twg, twu, tdy) = inputs(oracle, (1, 40, 64, 72), dtype, seed=13)
    tests = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_static")
    torch.library.opcheck(ops.swiglu_forward, (tx, twg, twu, True), test_utils=tests)
    torch.library.opcheck(ops.swiglu_forward, (tx.clone().requires_grad_(True), twg, twu.clone().requires_grad_(True), True),
                          test_utils=tests)
    _, g, u = ops.swiglu_forward(tx, twg, twu, True)
    for flags in ((True, True, True, False), (True, False, True, False), (False, True, True, True)):
        torch.library.opcheck(ops.swiglu_backward, (tdy, tx, twg, twu, g, u) + flags, test_utils=tests[:3])


def test_needs_input_grad_subsets(oracle):
    dtype = torch.float16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = inputs(oracle, (1, 64, 128, 136), dtype, seed=14)
    twu = twu.clone().requires_grad_(True)
    out = fsw.swiglu(tx, twg, twu, autocast_dtype=dtype)
    out.backward(tdy)
    torch.cuda.synchronize()
    assert tx.grad is None and twg.grad is None
    assert oracle.rel_error(np64(twu.grad), oracle.swiglu_backward(x, wg, wu, dy)[2]) < TOL[dtype]


def test_autocast_casts_like_the_reference_functions(oracle):
    """Under CUDA autocast fp32 arguments are cast to the module's dtype (custom_fwd(cast_inputs=...),
    swiglu.py:18); outside autocast fp32 arguments are refused."""
    (x, wg, wu, _), (tx, twg, twu, _) = inputs(oracle, (1, 32, 64, 72), torch.bfloat16, seed=15)
    m = fsw.SwiGLU(64, 72, device=DEV)
    with torch.no_grad():
        m.w_gate.copy_(twg)
        m.w_up.copy_(twu)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = m(tx.float())
    assert out.dtype == torch.bfloat16
    assert oracle.rel_error(np64(out), oracle.fused_swiglu_fwd(x, wg, wu)[0]) < 1e-2
    with pytest.raises(AssertionError):
        m(tx.float())


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_torch_compile_keeps_the_operator_opaque(oracle, backend):
    """torch.compile traces through module and operator in one graph and reproduces the eager results and
    gradients exactly: with the aot_eager backend (no code generation) and with the default inductor
    backend, which has to treat the registered operators as opaque calls around its own generated code."""
    dtype, shape = torch.bfloat16, (2, 64, 128, 264)
    _, (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=16)
    m = fsw.SwiGLU(shape[2], shape[3], device=DEV)
    with torch.no_grad():
        m.w_gate.copy_(twg)
        m.w_up.copy_(twu)
    xe = tx.clone().requires_grad_(True)
    oe = m(xe)
    oe.backward(tdy)
    ge = [xe.grad.clone(), m.w_gate.grad.clone(), m.w_up.grad.clone()]
    m.zero_grad(set_to_none=True)
    torch._dynamo.reset()
    cm = torch.compile(m, backend=backend, fullgraph=True)
    xc = tx.clone().requires_grad_(True)
    oc = cm(xc)
    oc.backward(tdy)
    torch.cuda.synchronize()
    assert torch.equal(oc, oe)
    assert torch.equal(xc.grad, ge[0]) and torch.equal(m.w_gate.grad, ge[1]) and torch.equal(m.w_up.grad, ge[2])


# ---- backward without saved pre-activations -----------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(2, 136, 264, 520), (1, 300, 256, 384), (3, 50, 72, 65), (1, 7, 8, 8), (1, 257, 100, 130)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gating_grad_recompute_launcher(oracle, dtype, shape):
    """fsw_gating_grad_recompute against the oracle's gating gradient evaluated on the exact
    pre-activations (tiled kernel for 8-aligned shapes, edge-shape kernel otherwise)."""
    from fusedswiglu_amd.kernels import kernels_bf16, kernels_fp16
    k = kernels_bf16 if dtype == torch.bfloat16 else kernels_fp16
    (x, wg, wu, dy), (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=21)
    dU, dG = k.gating_grad_recompute(tdy, tx, twg, twu)
    torch.cuda.synchronize()
    _, g, u = oracle.fused_swiglu_fwd(x, wg, wu)
    o_dU, o_dG = oracle.elementwise_backward(dy, g, u)
    assert dU.shape == tdy.shape and dG.shape == tdy.shape
    assert oracle.rel_error(np64(dU), o_dU) < TOL[dtype] and oracle.rel_error(np64(dG), o_dG) < TOL[dtype]
    assert oracle.rel_error(np64(dU), o_dG) > 0.1  # (up, gate) order as in elementwise_backward


@pytest.mark.parametrize("packed", [False, True], ids=["two_weights", "packed"])
def test_recompute_backward_saves_no_preactivations(oracle, packed):
    dtype, shape = torch.bfloat16, (2, 136, 264, 520)
    (x, wg, wu, dy), (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=22)
    T, I = shape[0] * shape[1], shape[3]
    grads, saved_elems = {}, {}
    for recompute in (False, True):
        m = fsw.SwiGLU(shape[2], shape[3], dtype=dtype, device=DEV, packed=packed, recompute=recompute)
        with torch.no_grad():
            if packed:
                m.w_gate_up.copy_(torch.cat([twg, twu], dim=1))
            else:
                m.w_gate.copy_(twg)
                m.w_up.copy_(twu)
        xin = tx.clone().requires_grad_(True)
        sizes = []
        with torch.autograd.graph.saved_tensors_hooks(lambda t: (sizes.append(t.numel()), t)[1], lambda t: t):
            out = m(xin)
        out.backward(tdy)
        torch.cuda.synchronize()
        saved_elems[recompute] = sum(sizes)
        w = m.w_gate_up.grad if packed else torch.cat([m.w_gate.grad, m.w_up.grad], dim=1)
        grads[recompute] = (out.detach(), xin.grad, w)
    assert saved_elems[False] - saved_elems[True] == 2 * T * I
    o_out = oracle.fused_swiglu_fwd(x, wg, wu)[0]
    o_dx, o_dwg, o_dwu = oracle.swiglu_backward(x, wg, wu, dy)
    out, dx, dw = grads[True]
    assert torch.equal(out, grads[False][0])
    assert oracle.rel_error(np64(out), o_out) < 1e-2 and oracle.rel_error(np64(dx), o_dx) < 1e-2
    assert oracle.rel_error(np64(dw[:, :I]), o_dwg) < 1e-2 and oracle.rel_error(np64(dw[:, I:]), o_dwu) < 1e-2
    # recomputed pre-activations are not rounded to 16 bits first: not worse than the saving path
    assert oracle.rel_error(np64(dx), o_dx) <= 1.05 * oracle.rel_error(np64(grads[False][1]), o_dx)


def test_hip_graph_capture_and_replay(oracle):
    """The whole forward + backward captured into one HIP graph (the library only enqueues kernels on
    the given stream, never allocates or synchronises): every replay, with fresh input values copied
    into the captured buffers and eager work in between, reproduces the eager result bit for bit."""
    dtype, shape = torch.bfloat16, (2, 192, 256, 768)   # small d_model: the split-reduction path with its scratch
    _, (tx, twg, twu, tdy) = inputs(oracle, shape, dtype, seed=31)
    sx = tx.clone().requires_grad_(True)
    swg = twg.clone().requires_grad_(True)
    swu = twu.clone().requires_grad_(True)
    sdy = tdy.clone()

    def step():
        out = fsw.FusedSwiGLU.apply(sx, swg, swu)
        gx, gwg, gwu = torch.autograd.grad(out, (sx, swg, swu), sdy)
        return out, gx, gwg, gwu

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(3):
        scale = 1.0 + 0.5 * rep
        with torch.no_grad():
            sx.copy_(tx * scale)
            sdy.copy_(tdy * (2.0 - 0.25 * rep))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()                      # eager, on the current stream, between replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)
