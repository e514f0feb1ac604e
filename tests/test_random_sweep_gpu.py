"""Seeded random sweep over everything a caller can vary at once: token count (1 .. 5000, so the weight-streaming,
eight-wave, four-wave, split-reduction and edge kernels all take their turn), dimensions that are and are not
multiples of 8, either weight layout, either element type, leading dimensions larger than the row length, with and
without stored pre-activations, the down projection in either storage order behind it.  Every launcher runs through
the C ABI and is compared with an fp32 product of the same (rounded) operands on the GPU; the first cases of every
seed are small enough for the CPU oracle and are checked against it too, which ties the fp32 products used here to
the oracle of the other tests.  Metric and bounds: rel-L2 <= 1e-2 for bfloat16 (fused_swiglu/test_swiglu.py:20),
<= 5e-3 for float16."""
import random

import numpy as np
import pytest
import torch

from fusedswiglu_amd.kernels import _launch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.bfloat16: 1e-2, torch.float16: 5e-3}
NAME = {torch.bfloat16: "bf16", torch.float16: "fp16"}
CASES_PER_SEED = 40


def rel(a, r):
    a, r = a.float(), r.float()
    if not bool(torch.isfinite(a).all()):
        return float("inf")
    return ((a - r).norm() / (r.norm() + 1e-30)).item()


def np64(t):
    return t.detach().float().cpu().double().numpy()


def pick_dim(rng, big):
    r = rng.random()
    if r < 0.15:
        return rng.randint(1, 300)            # any value: the edge kernel
    if r < 0.75:
        return 8 * rng.randint(1, 160)
    return 8 * rng.randint(160, big // 8)


def pick_tokens(rng):
    r = rng.random()
    if r < 0.2:
        return rng.randint(1, 16)
    if r < 0.4:
        return rng.randint(17, 128)
    if r < 0.6:
        return rng.randint(129, 256)
    if r < 0.9:
        return rng.randint(257, 1500)
    return 8 * rng.randint(256, 640)


def strided(rows, cols, dtype, scale, pad):
    """[rows, cols] with a leading dimension of cols + pad"""
    full = (torch.randn(rows, cols + pad, device=DEV) * scale).to(dtype)
    return full[:, :cols] if pad else full


@pytest.mark.parametrize("seed", range(8))
def test_every_launcher_on_random_shapes_layouts_and_strides(oracle, seed):
    rng = random.Random(7000 + seed)
    torch.manual_seed(7000 + seed)
    for ci in range(CASES_PER_SEED):
        dtype = rng.choice([torch.bfloat16, torch.float16])
        out_in = rng.random() < 0.5
        T, D, I = pick_tokens(rng), pick_dim(rng, 4608), pick_dim(rng, 3072)
        if ci < 3:  # small enough for the oracle
            T, D, I = min(T, 300), min(D, 520), min(I, 520)
        if T * D * I > 3e9:
            T = max(1, int(3e9 / (D * I)))
        padx, padw = rng.choice([0, 0, 8, 24]), rng.choice([0, 0, 8, 40])
        save = rng.random() < 0.7
        case = f"seed {seed} case {ci}: {NAME[dtype]} T={T} D={D} I={I} out_in={out_in} padx={padx} padw={padw} save={save}"
        print(case, flush=True)
        tol = TOL[dtype]
        x = strided(T, D, dtype, 1.0, padx)
        wrows, wcols = (I, D) if out_in else (D, I)
        wg, wu = strided(wrows, wcols, dtype, D ** -0.5, padw), strided(wrows, wcols, dtype, D ** -0.5, padw)
        dy = torch.randn(T, I, device=DEV).to(dtype)
        wgf, wuf = (wg.float().t(), wu.float().t()) if out_in else (wg.float(), wu.float())
        rg, ru = x.float() @ wgf, x.float() @ wuf

        out, g, u = _launch.fused_swiglu_fwd(x, wg, wu, dtype, save_preactivations=save, weights_out_in=out_in)
        assert rel(out, torch.nn.functional.silu(rg) * ru) < tol, case
        if save:
            assert rel(g, rg) < tol and rel(u, ru) < tol, case
        else:
            assert g is None and u is None, case
            g, u = rg.to(dtype), ru.to(dtype)
        # the gating gradient from the stored (rounded) pre-activations, and from x and the weights
        gf, uf, dyf = g.float(), u.float(), dy.float()
        s = torch.sigmoid(gf)
        dU, dG = _launch.elementwise_backward(dy, g, u, dtype)
        assert rel(dU, dyf * gf * s) < tol and rel(dG, dyf * uf * (s + gf * s * (1 - s))) < tol, case
        dU2, dG2 = _launch.gating_grad_recompute(dy, x, wg, wu, dtype, weights_out_in=out_in)
        s2 = torch.sigmoid(rg)
        assert rel(dU2, dyf * rg * s2) < tol and rel(dG2, dyf * ru * (s2 + rg * s2 * (1 - s2))) < tol, case
        # the two gradient GEMMs on the rounded gating gradients, and the one-call backward bit for bit
        dx = _launch.fused_input_grad(dG, dU, wg, wu, dtype, weights_out_in=out_in)
        assert rel(dx, dG.float() @ wgf.t() + dU.float() @ wuf.t()) < tol, case
        dWu, dWg = _launch.fused_weight_grad(x, dU, dG, dtype, weights_out_in=out_in)
        rWg, rWu = x.float().t() @ dG.float(), x.float().t() @ dU.float()
        assert rel(dWg, rWg.t() if out_in else rWg) < tol and rel(dWu, rWu.t() if out_in else rWu) < tol, case
        bx, bwg, bwu = _launch.swiglu_backward(dy, x, wg, wu, g, u, dtype, weights_out_in=out_in)
        assert torch.equal(bx, dx) and torch.equal(bwg, dWg) and torch.equal(bwu, dWu), case

        if ci < 3:
            ox, owg, owu = np64(x), np64(wgf), np64(wuf)
            o_out, o_g, o_u = oracle.fused_swiglu_fwd(ox, owg, owu)
            assert oracle.rel_error(np64(out), o_out) < tol, case
            o_dx, o_dwg, o_dwu = oracle.swiglu_backward(ox, owg, owu, np64(dy))
            # the oracle keeps g and u in full precision: its gradients differ from the path's by their rounding
            assert oracle.rel_error(np64(dx), o_dx) < 2 * tol, case
            assert oracle.rel_error(np64(dWg.t() if out_in else dWg), o_dwg) < 2 * tol, case
            assert oracle.rel_error(np64(dWu.t() if out_in else dWu), o_dwu) < 2 * tol, case

        if rng.random() < 0.5:   # the down projection behind it
            Dd, down_out_in = pick_dim(rng, 2048), rng.random() < 0.5
            wd = strided(Dd if down_out_in else I, I if down_out_in else Dd, dtype, I ** -0.5, rng.choice([0, 8]))
            wdf = wd.float().t() if down_out_in else wd.float()
            case += f" down to {Dd} out_in={down_out_in}"
            y = _launch.down_proj_forward(out, wd, dtype, weights_out_in=down_out_in)
            assert rel(y, out.float() @ wdf) < tol, case
            gy = torch.randn(T, Dd, device=DEV).to(dtype)
            da = _launch.down_proj_input_grad(gy, wd, dtype, weights_out_in=down_out_in)
            assert rel(da, gy.float() @ wdf.t()) < tol, case
            dwd = _launch.down_proj_weight_grad(out, gy, dtype, weights_out_in=down_out_in)
            rwd = out.float().t() @ gy.float()
            assert rel(dwd, rwd.t() if down_out_in else rwd) < tol, case
    torch.cuda.synchronize()
