"""CPU-only checks of the C-ABI library and the host logic: the library loads, exports every
symbol the header declares, validates its arguments before touching the GPU, and the Python
boundary raises the reference's kind of errors.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

from fusedswiglu_amd import FastAccumFusedSwiGLU, FusedSwiGLU, _abi
from fusedswiglu_amd.kernels import kernels_bf16, kernels_fp16

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(_abi.LIBRARY_PATH):
        _abi.build_library()
    return _abi.lib()


def _declared(header_name):
    header = open(os.path.join(ROOT, "include", header_name)).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    return set(re.findall(r"\b(fsw_[a-z_0-9]+)\s*\(", header))


def _exported(path):
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", path], stdout=subprocess.PIPE, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line}


def test_header_symbols_all_exported(L):
    """The drop-in library exports exactly what include/fusedswiglu.h declares - the path and nothing else;
    the benchmark probes live in a library and a header of their own."""
    declared = _declared("fusedswiglu.h")
    assert declared == set(_abi.EXPORTED_SYMBOLS)
    assert _exported(_abi.LIBRARY_PATH) == declared
    for name in declared:
        assert getattr(L, name) is not None
    header = open(os.path.join(ROOT, "include", "fusedswiglu.h")).read()
    m = re.search(r"#define FSW_VERSION (\d+)", header)
    assert L.fsw_version() == int(m.group(1)) == 400   # 0.4.0: the backward in one call
    assert "probe" not in header and "force_edge" not in header
    bench = _declared("fusedswiglu_bench.h")
    assert bench == set(_abi.BENCH_SYMBOLS) == _exported(_abi.BENCH_LIBRARY_PATH)
    for name in bench:
        assert getattr(_abi.bench_lib(), name) is not None


def test_status_strings(L):
    assert L.fsw_status_string(0) == b"ok"
    seen = {L.fsw_status_string(i) for i in range(0, 8)}
    assert len(seen) == 8
    assert L.fsw_status_string(99) == b"unknown status"


P = ctypes.c_void_p(0x1000)  # a fake, aligned, non-null "device pointer": never dereferenced here


def test_forward_validation(L):
    f = L.fsw_swiglu_forward
    assert f(None, P, P, P, P, P, 8, 8, 8, 8, 8, 8, 0, None) == 1
    assert b"non-null" in L.fsw_last_error()
    assert f(P, P, P, P, P, None, 8, 8, 8, 8, 8, 8, 0, None) == 1  # only one of g/u
    assert f(P, P, P, P, P, P, 8, 8, 8, 8, 8, 8, 7, None) == 2
    assert f(P, P, P, P, P, P, 0, 8, 8, 8, 8, 8, 0, None) == 3
    assert f(P, P, P, P, P, P, 8, -1, 8, 8, 8, 8, 0, None) == 3
    assert f(P, P, P, P, P, P, 2 ** 31, 8, 8, 8, 8, 8, 0, None) == 3
    assert f(P, P, P, P, P, P, 8, 8, 8, 7, 8, 8, 0, None) == 4  # ldx < D
    assert f(P, P, P, P, P, P, 8, 8, 16, 8, 8, 16, 1, None) == 4  # ldw < I
    assert f(P, P, P, P, P, P, 8, 8, 16, 8, 16, 8, 1, None) == 4  # ldo < I
    assert f(ctypes.c_void_p(0x1001), P, P, P, P, P, 8, 8, 8, 8, 8, 8, 0, None) == 5
    assert L.fsw_last_error() != b""


def test_backward_validation(L):
    e = L.fsw_elementwise_backward
    assert e(P, P, None, P, P, 8, 0, None) == 1
    assert e(P, P, P, P, P, 0, 0, None) == 3
    assert e(P, P, P, P, P, 8, 2, None) == 2
    rc = L.fsw_gating_grad_recompute
    assert rc(P, P, P, None, P, P, 8, 8, 8, 8, 8, 8, 0, None) == 1
    assert rc(P, P, P, P, P, P, 8, 8, 8, 8, 8, 8, 5, None) == 2
    assert rc(P, P, P, P, P, P, 8, 0, 8, 8, 8, 8, 0, None) == 3
    assert rc(P, P, P, P, P, P, 8, 8, 16, 8, 16, 8, 0, None) == 4  # ldo < I
    assert rc(P, P, P, ctypes.c_void_p(0x1001), P, P, 8, 8, 8, 8, 8, 8, 0, None) == 5
    # the backward in one call validates all three steps before it launches the first
    bw = L.fsw_swiglu_backward
    ok_dims = (8, 8, 8, 8, 8, 8, 8)                                    # T, D, I, ldx, ldw, ld_dx, ld_dw
    assert bw(P, P, None, P, P, P, P, P, P, P, P, *ok_dims, None, 0, 0, None) == 1          # no xw_up
    assert bw(P, P, P, P, P, P, P, P, P, P, None, *ok_dims, None, 0, 0, None) == 1          # one weight gradient only
    assert bw(P, P, P, P, None, P, P, P, P, P, P, *ok_dims, None, 0, 0, None) == 1          # grad_x without w_gate
    assert bw(P, P, P, None, P, P, P, P, None, P, P, *ok_dims, None, 0, 0, None) == 1       # weight gradients without x
    assert bw(P, P, P, P, P, P, P, P, P, P, P, 8, 8, 8, 8, 8, 4, 8, None, 0, 0, None) == 4  # ld_dx < D
    assert bw(P, P, P, P, P, P, P, P, P, P, P, 8, 8, 16, 8, 16, 8, 8, None, 0, 0, None) == 4  # ld_dw < I
    assert bw(P, P, P, P, P, P, P, P, P, P, P, 8, 16, 8, 8, 8, 16, 8, None, 0, 0, None) == 4  # ldx < D
    assert bw(P, P, P, P, P, P, P, P, P, P, P, 0, 8, 8, 8, 8, 8, 8, None, 0, 0, None) == 3
    assert bw(P, P, P, P, P, P, P, P, P, P, P, *ok_dims, None, 0, 4, None) == 2
    assert bw(ctypes.c_void_p(0x1001), P, P, P, P, P, P, P, P, P, P, *ok_dims, None, 0, 0, None) == 5
    dx = L.fsw_input_grad
    assert dx(P, P, P, P, None, 8, 8, 8, 8, 8, 8, None, 0, 0, None) == 1
    assert dx(P, P, P, P, P, 8, 8, 8, 8, 8, 4, None, 0, 0, None) == 4  # ld_dx < D
    assert dx(P, P, P, P, P, 8, 8, 0, 8, 8, 8, None, 0, 0, None) == 3
    # the variant on the library's built-in scratch validates the same way, and turns problems whose split
    # reduction needs more than that buffer away before it touches the GPU
    na = L.fsw_input_grad_noalloc
    assert na(P, P, P, P, None, 8, 8, 8, 8, 8, 8, 0, None) == 1
    assert na(P, P, P, P, P, 8, 8, 8, 8, 8, 4, 0, None) == 4
    assert na(P, P, P, P, P, 8, 8, 8, 8, 8, 8, 9, None) == 2
    assert L.fsw_workspace_bytes(1, 16384, 256, 2048) > _abi.NOALLOC_SCRATCH_BYTES
    assert na(P, P, P, P, P, 16384, 256, 2048, 2048, 2048, 256, 0, None) == _abi.ERR_SCRATCH_LIMIT
    assert b"built-in buffer" in L.fsw_last_error()
    header = open(os.path.join(ROOT, "include", "fusedswiglu.h")).read()
    assert re.search(r"#define FSW_NOALLOC_SCRATCH_BYTES \(32u << 20\)", header) and _abi.NOALLOC_SCRATCH_BYTES == 32 << 20
    # the weight-layout flag rides on dtype: it changes which dimension ldw / ld_dw must cover
    OI = _abi.WEIGHTS_OUT_IN
    f = L.fsw_swiglu_forward
    assert f(P, P, P, P, P, P, 8, 8, 16, 8, 8, 16, 0 | OI, None) != 4    # [I,D] weights: ldw >= D = 8 is enough
    assert f(P, P, P, P, P, P, 8, 16, 8, 16, 8, 8, 0 | OI, None) == 4    # ldw = 8 < D = 16
    assert f(P, P, P, P, P, P, 8, 8, 8, 8, 8, 8, 0x200, None) == 2       # unknown flag
    assert dx(P, P, P, P, P, 8, 16, 8, 8, 8, 16, None, 0, 1 | OI, None) == 4  # ldw < D
    dn = L.fsw_down_proj_forward
    assert dn(P, None, P, 8, 8, 8, 8, 8, 8, None, 0, 0, None) == 1
    assert dn(P, P, P, 8, 16, 8, 16, 4, 8, None, 0, 0, None) == 4          # w_down [I,D]: ldw < D
    assert dn(P, P, P, 8, 16, 8, 16, 8, 8, None, 0, OI, None) == 4         # w_down [D,I]: ldw < I
    assert dn(P, P, P, 8, 16, 8, 8, 8, 8, None, 0, 0, None) == 4           # ld_act < I
    assert L.fsw_down_proj_input_grad(P, P, P, 8, 8, 0, 8, 8, 8, None, 0, 0, None) == 3
    assert L.fsw_down_proj_weight_grad(P, P, P, 8, 8, 8, 8, 8, 8, None, 0, 5, None) == 2
    # few output tiles and long reductions ask for scratch in the down projection's gradients too
    assert L.fsw_workspace_bytes(6, 8192, 256, 768) > 0 and L.fsw_workspace_bytes(6 | OI, 8192, 256, 768) > 0
    assert L.fsw_workspace_bytes(4, 8192, 4096, 12288) == 0 and L.fsw_workspace_bytes(2 | OI, 8192, 4096, 12288) == 0
    dw = L.fsw_weight_grad
    assert dw(P, None, P, P, P, 8, 8, 8, 8, 8, 8, None, 0, 1, None) == 1
    assert dw(P, P, P, P, P, 8, 8, 8, 8, 8, 8, None, 0, -3, None) == 2
    assert dw(P, P, P, P, P, 8, 16, 8, 8, 8, 8, None, 0, 1, None) == 4  # ldx < D
    # small d_model: few output tiles, long reductions -> the library asks for split-K scratch
    assert L.fsw_workspace_bytes(1, 8192, 256, 768) % (8192 * 256 * 4) == 0 and L.fsw_workspace_bytes(1, 8192, 256, 768) > 0
    assert L.fsw_workspace_bytes(2, 8192, 256, 768) % (2 * 256 * 768 * 4) == 0 and L.fsw_workspace_bytes(2, 8192, 256, 768) > 0
    # the headline shape fills the chip: no scratch
    assert L.fsw_workspace_bytes(1, 8192, 4096, 12288) == 0 and L.fsw_workspace_bytes(2, 8192, 4096, 12288) == 0
    assert L.fsw_workspace_bytes(0, 8192, 256, 768) == 0 and L.fsw_workspace_bytes(1, 0, 1, 1) == 0


def test_probe_validation():
    L = _abi.bench_lib()
    f = L.fsw_probe_mfma_mix
    flop = ctypes.c_double(0.0)
    assert f(1, 10, 256, None, 8 << 20, P, None, ctypes.byref(flop)) == 3          # no source window
    assert f(1, 10, 256, P, (8 << 20) + 4096, P, None, ctypes.byref(flop)) == 3    # not a multiple of 256 KiB
    assert f(1, 10, 256, P, 1 << 31, P, None, ctypes.byref(flop)) == 3             # beyond the descriptor's reach
    assert f(9, 10, 256, P, 8 << 20, P, None, ctypes.byref(flop)) == 3             # unknown mix
    assert f(1, 0, 256, P, 8 << 20, P, None, ctypes.byref(flop)) == 3
    assert L.fsw_probe_mfma(1, 0, 256, P, None, ctypes.byref(flop)) == 3
    assert L.fsw_probe_stream_read(None, 1 << 20, P, None) == 3


def test_kernel_selection_logic(L):
    t = L.fsw_uses_tiled_kernel
    # the north-star shape and the fp16 config run on the tiled kernels in all three steps
    for step in range(4):
        assert t(step, 8192, 4096, 12288, 4096, 12288, 12288, 4096 if step == 1 else 12288, 16) == 1
        assert t(step, 8192, 4096, 11008, 4096, 11008, 11008, 4096 if step == 1 else 11008, 16) == 1
    assert t(3, 8192, 4096, 11007, 4096, 11007, 11007, 11007, 16) == 0 and t(7, 8, 8, 8, 8, 8, 8, 8, 16) == 0
    # the down projection (steps 4 / 5 / 6; ldx: [T,D] arrays, ldw: W_down, ldo: [T,I] arrays): tiled for many
    # tokens, weight streaming up to 128 tokens when half the result columns are aligned, never for the weight
    # gradient; W_down [I,D] by default, [D,I] with the layout flag
    OI = 0x100
    for step in (4, 5, 6):
        assert t(step, 8192, 4096, 12288, 4096, 4096, 12288, 4096, 16) == 1
        assert t(step | OI, 8192, 4096, 12288, 4096, 12288, 12288, 12288, 16) == 1
        assert t(step, 8192, 4096, 12281, 4096, 4096, 12281, 4096, 16) == 0
    assert t(4, 16, 8192, 28672, 8192, 8192, 28672, 8192, 16) == 2 and t(4 | OI, 128, 8192, 28672, 8192, 28672, 28672, 28672, 16) == 2
    assert t(5, 16, 8192, 28672, 8192, 8192, 28672, 8192, 16) == 2 and t(6, 16, 8192, 28672, 8192, 8192, 28672, 8192, 16) == 1
    assert t(5, 16, 8192, 72, 8192, 8192, 72, 8192, 16) == 1 and t(5 | OI, 16, 8192, 136, 8192, 136, 136, 136, 16) == 1
    assert t(4, 129, 8192, 28672, 8192, 8192, 28672, 8192, 16) == 1
    # dimensions that are not multiples of 8, or unaligned pointers, take the edge-shape kernel
    assert t(0, 8192, 4096, 11007, 4096, 11007, 11007, 11007, 16) == 0
    assert t(0, 8192, 4100, 12288, 4100, 12288, 12288, 12288, 16) == 0
    assert t(0, 8192, 4096, 12288, 4096, 12288, 12288, 12288, 2) == 0
    # the token count is free: it is never the contiguous index of an operand
    assert t(0, 8191, 4096, 12288, 4096, 12288, 12288, 12288, 16) == 1
    assert t(2, 8191, 4096, 12288, 4096, 12288, 12288, 12288, 16) == 1
    # few tokens: the forward streams the weights once with its own kernel (only the forward)
    assert t(0, 128, 8192, 28672, 8192, 28672, 28672, 28672, 16) == 2 and t(0, 16, 8192, 28672, 8192, 28672, 28672, 28672, 16) == 2
    assert t(0, 129, 8192, 28672, 8192, 28672, 28672, 28672, 16) == 1 and t(3, 16, 8192, 28672, 8192, 28672, 28672, 28672, 16) == 1
    assert t(0, 16, 8192, 28672, 8192, 28672, 28672, 28672, 2) == 0
    # result rows are indexed through a 32-bit leading dimension on the tiled kernels: beyond that, edge kernel
    assert t(0, 8, 64, 64, 64, 64, 2 ** 31, 64, 16) == 0 and t(1, 512, 64, 64, 64, 64, 64, 2 ** 31 + 8, 16) == 0


def test_python_boundary_errors_without_gpu():
    """Shape / dtype / device problems raise before any launch, as AssertionError like the
    reference's asserts (fused_swiglu/kernels/kernels_bf16.py:170-182) and as ValueError."""
    bf = torch.bfloat16
    x = torch.zeros(2, 4, 8, dtype=bf)
    w = torch.zeros(8, 16, dtype=bf)
    with pytest.raises(AssertionError, match="Dimension mismatch"):
        kernels_bf16.fused_swiglu_fwd(x, torch.zeros(9, 16, dtype=bf), torch.zeros(9, 16, dtype=bf))
    with pytest.raises(ValueError, match="same shape"):
        kernels_bf16.fused_swiglu_fwd(x, w, torch.zeros(8, 24, dtype=bf))
    with pytest.raises(AssertionError, match="number of dimensions"):
        kernels_bf16.fused_swiglu_fwd(x, w[None], w[None])
    with pytest.raises(AssertionError, match="bfloat16"):
        kernels_bf16.fused_swiglu_fwd(x.float(), w.float(), w.float())
    with pytest.raises(AssertionError, match="float16"):
        kernels_fp16.fused_swiglu_fwd(x, w, w)
    # right shapes and dtype but host tensors: refused, never computed on the CPU
    with pytest.raises(AssertionError, match="HIP GPU"):
        kernels_bf16.fused_swiglu_fwd(x, w, w)
    with pytest.raises(AssertionError, match="HIP GPU"):
        FusedSwiGLU.apply(x, w, w)
    with pytest.raises(AssertionError, match="HIP GPU"):
        FastAccumFusedSwiGLU.apply(x.half().requires_grad_(), w.half(), w.half())
    with pytest.raises(AssertionError, match="same shape"):
        kernels_bf16.elementwise_backward(torch.zeros(2, 3, dtype=bf), torch.zeros(2, 4, dtype=bf), torch.zeros(2, 3, dtype=bf))


def test_package_exports():
    import fusedswiglu_amd

    # the reference's two names first (fused_swiglu/__init__.py:1-2), then this build's additions
    assert fusedswiglu_amd.__all__[:2] == ["FusedSwiGLU", "FastAccumFusedSwiGLU"]
    assert set(fusedswiglu_amd.__all__[2:]) == {"swiglu", "swiglu_packed", "down_proj", "swiglu_mlp", "SwiGLU", "SwiGLUMLP"}
    assert issubclass(FusedSwiGLU, torch.autograd.Function)
    assert issubclass(FastAccumFusedSwiGLU, torch.autograd.Function)


def test_product_does_not_import_oracle():
    """The oracle is test infrastructure: nothing under the package may reference it."""
    pkg = os.path.join(ROOT, "fusedswiglu_amd")
    for dirpath, _, files in os.walk(pkg):
        for fn in files:
            if fn.endswith((".py", ".hip", ".hpp", ".h", "Makefile")):
                text = open(os.path.join(dirpath, fn)).read()
                assert "oracle" not in text.lower(), f"{fn} mentions the oracle"
