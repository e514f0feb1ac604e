"""The entry point that allocates nothing, fsw_input_grad_noalloc, against fsw_input_grad with a caller
workspace: same split plan, same kernels, so the results must be bit-identical.  Two calls in a row on the
library's built-in scratch, the second with a smaller input; then the oracle on the smaller one.  The file is
named so that pytest collects it last."""
import ctypes

import numpy as np
import pytest
import torch

from fusedswiglu_amd import _abi

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TORCH = {"bf16": torch.bfloat16, "fp16": torch.float16}
CODE = {"bf16": _abi.DTYPE_BF16, "fp16": _abi.DTYPE_FP16}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _inputs(T, D, I, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    dG = torch.randn(T, I, generator=g).to(DEV).to(dtype)
    dU = torch.randn(T, I, generator=g).to(DEV).to(dtype)
    wg = (torch.randn(D, I, generator=g) / D ** 0.5).to(DEV).to(dtype)
    wu = (torch.randn(D, I, generator=g) / D ** 0.5).to(DEV).to(dtype)
    return dG, dU, wg, wu


def _with_workspace(dG, dU, wg, wu, code):
    T, I = dG.shape
    D = wg.shape[0]
    L = _abi.lib()
    need = L.fsw_workspace_bytes(_abi.STEP_INPUT_GRAD, T, D, I)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    dx = torch.full((T, D), float("nan"), dtype=dG.dtype, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _abi.check(L.fsw_input_grad(_ptr(dG), _ptr(dU), _ptr(wg), _ptr(wu), _ptr(dx), T, D, I, I, I, D,
                                _ptr(ws), need, code, stream))
    return dx, need


def _no_alloc(dG, dU, wg, wu, code):
    T, I = dG.shape
    D = wg.shape[0]
    dx = torch.full((T, D), float("nan"), dtype=dG.dtype, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _abi.check(_abi.lib().fsw_input_grad_noalloc(_ptr(dG), _ptr(dU), _ptr(wg), _ptr(wu), _ptr(dx), T, D, I,
                                                 I, I, D, code, stream))
    return dx


@pytest.mark.parametrize("name", ["bf16", "fp16"])
def test_no_alloc_input_grad_matches_workspace_variant(name, oracle):
    dtype, code = TORCH[name], CODE[name]
    # both problems split their reduction (few output tiles, long reduction) and fit the built-in scratch
    shapes = [(2048, 256, 2048), (1000, 128, 1536)]
    results = []
    for seed, (T, D, I) in enumerate(shapes):
        dG, dU, wg, wu = _inputs(T, D, I, dtype, seed)
        want, need = _with_workspace(dG, dU, wg, wu, code)
        assert 0 < need <= _abi.NOALLOC_SCRATCH_BYTES, "the case is meant to use the split reduction"
        got = _no_alloc(dG, dU, wg, wu, code)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"call {seed}: T={T} D={D} I={I}"
        results.append((got, dG, dU, wg, wu))
    # the second, smaller call against the oracle (bound as in the parity tests)
    got, dG, dU, wg, wu = results[1]
    f64 = lambda t: t.float().cpu().double().numpy()
    ref = oracle.input_grad(f64(dG), f64(dU), f64(wg), f64(wu))
    err = np.linalg.norm(f64(got) - ref) / np.linalg.norm(ref)
    assert err <= (1e-2 if name == "bf16" else 5e-3), err


def test_no_alloc_large_problem_needs_no_scratch():
    # plenty of output tiles: no split, the built-in buffer is not touched, results equal the plain call
    dG, dU, wg, wu = _inputs(8192, 8192, 64, torch.bfloat16, 7)
    want, need = _with_workspace(dG, dU, wg, wu, _abi.DTYPE_BF16)
    assert need == 0
    got = _no_alloc(dG, dU, wg, wu, _abi.DTYPE_BF16)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_no_alloc_skips_a_tail_split_that_does_not_fit():
    # 39 x 9 = 351 output tiles: one full round of 256 and a tail of 95, whose split would take 47.5 MiB of partial
    # tiles.  With the caller's large workspace fsw_input_grad splits the tail; the built-in 32 MiB do not hold it,
    # so this call runs the tail unsplit: bit-identical to fsw_input_grad given 32 MiB, and equal to the split
    # result up to the order of the fp32 sums (same distance from an fp32 product).
    T, D, I = 9984, 2304, 2608
    dG, dU, wg, wu = _inputs(T, D, I, torch.float16, 11)
    split, need = _with_workspace(dG, dU, wg, wu, _abi.DTYPE_FP16)
    assert need > _abi.NOALLOC_SCRATCH_BYTES, "the case is meant to ask for more than the built-in scratch"
    got = _no_alloc(dG, dU, wg, wu, _abi.DTYPE_FP16)
    ws = torch.empty(_abi.NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device=DEV)
    same_plan = torch.full((T, D), float("nan"), dtype=torch.float16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _abi.check(_abi.lib().fsw_input_grad(_ptr(dG), _ptr(dU), _ptr(wg), _ptr(wu), _ptr(same_plan), T, D, I, I, I, D,
                                         _ptr(ws), _abi.NOALLOC_SCRATCH_BYTES, _abi.DTYPE_FP16, stream))
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), same_plan.view(torch.int16))
    ref = dG.float() @ wg.float().t() + dU.float() @ wu.float().t()
    err = lambda a: float((a.float() - ref).norm() / ref.norm())
    assert err(got) < 5e-3 and abs(err(got) - err(split)) < 1e-6, (err(got), err(split))
    assert float((got != split).float().mean()) < 1e-2   # a few last bits, not a different result


def test_no_alloc_rejects_problems_beyond_the_built_in_scratch():
    T, D, I = 16384, 256, 2048
    L = _abi.lib()
    assert L.fsw_workspace_bytes(_abi.STEP_INPUT_GRAD, T, D, I) > _abi.NOALLOC_SCRATCH_BYTES
    dG, dU, wg, wu = _inputs(T, D, I, torch.bfloat16, 3)
    dx = torch.zeros(T, D, dtype=torch.bfloat16, device=DEV)
    status = L.fsw_input_grad_noalloc(_ptr(dG), _ptr(dU), _ptr(wg), _ptr(wu), _ptr(dx), T, D, I, I, I, D,
                                      _abi.DTYPE_BF16, None)
    assert status == _abi.ERR_SCRATCH_LIMIT
    assert b"built-in buffer" in L.fsw_last_error()
    torch.cuda.synchronize()
    assert float(dx.float().abs().max()) == 0.0  # nothing was enqueued
