"""ctypes binding of libfusedswiglu (the C ABI declared in include/fusedswiglu.h).

The library is built in-tree (fusedswiglu_amd/csrc/libfusedswiglu.so) by `build_library()`
or `make -C fusedswiglu_amd/csrc`.  There is no CPU fallback: if the library is missing or
a call fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import threading

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIBRARY_PATH = os.path.join(_CSRC, "libfusedswiglu.so")
#: machine probes for the benchmark harness: a separate library, not part of the drop-in boundary
BENCH_LIBRARY_PATH = os.path.join(_CSRC, "libfusedswiglu_bench.so")

DTYPE_BF16 = 0
DTYPE_FP16 = 1
#: OR-ed into a dtype code (or a workspace step): weights are stored "out x in" like nn.Linear.weight
WEIGHTS_OUT_IN = 0x100
STEP_DOWN_FORWARD, STEP_DOWN_INPUT_GRAD, STEP_DOWN_WEIGHT_GRAD = 4, 5, 6

STEP_FORWARD, STEP_INPUT_GRAD, STEP_WEIGHT_GRAD = 0, 1, 2

#: size of the scratch built into the library for fsw_input_grad_noalloc (FSW_NOALLOC_SCRATCH_BYTES)
NOALLOC_SCRATCH_BYTES = 32 << 20
ERR_SCRATCH_LIMIT = 7

#: every symbol include/fusedswiglu.h declares
EXPORTED_SYMBOLS = (
    "fsw_version",
    "fsw_status_string",
    "fsw_last_error",
    "fsw_uses_tiled_kernel",
    "fsw_workspace_bytes",
    "fsw_swiglu_forward",
    "fsw_elementwise_backward",
    "fsw_gating_grad_recompute",
    "fsw_input_grad",
    "fsw_input_grad_noalloc",
    "fsw_weight_grad",
    "fsw_swiglu_backward",
    "fsw_down_proj_forward",
    "fsw_down_proj_input_grad",
    "fsw_down_proj_weight_grad",
)
#: every symbol include/fusedswiglu_bench.h declares (libfusedswiglu_bench.so)
BENCH_SYMBOLS = ("fsw_probe_mfma", "fsw_probe_stream_read", "fsw_probe_mfma_mix", "fsw_probe_dma_read")


class FusedSwiGLUError(RuntimeError):
    """A libfusedswiglu call returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"libfusedswiglu status {status}: {message}")
        self.status = status


class LibraryNotBuiltError(ImportError):
    """libfusedswiglu.so is missing: the HIP extension was not built."""


_lib = None
_lock = threading.Lock()


def build_library(verbose: bool = False, jobs: int = 4) -> str:
    """Compile the HIP sources for gfx950 with hipcc (works without a GPU) and return the
    path of the shared library.  Always recompiles."""
    global _lib, _bench_lib
    cmd = ["make", "-C", _CSRC, f"-j{jobs}", "-B"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libfusedswiglu.so failed")
    _lib = None
    _bench_lib = None
    return LIBRARY_PATH


def lib() -> ctypes.CDLL:
    """The loaded library with argument types set.  Raises LibraryNotBuiltError if absent."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIBRARY_PATH):
            raise LibraryNotBuiltError(
                f"{LIBRARY_PATH} not found; build it with `make -C {_CSRC}` "
                "(or fusedswiglu_amd._abi.build_library()). There is no fallback path."
            )
        L = ctypes.CDLL(LIBRARY_PATH)
        vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.fsw_version.restype = ci
        L.fsw_version.argtypes = []
        L.fsw_status_string.restype = ctypes.c_char_p
        L.fsw_status_string.argtypes = [ci]
        L.fsw_last_error.restype = ctypes.c_char_p
        L.fsw_last_error.argtypes = []
        L.fsw_uses_tiled_kernel.restype = ci
        L.fsw_uses_tiled_kernel.argtypes = [ci, i64, i64, i64, i64, i64, i64, i64, ctypes.c_uint]
        L.fsw_swiglu_forward.restype = ci
        L.fsw_swiglu_forward.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, vp]
        L.fsw_elementwise_backward.restype = ci
        L.fsw_elementwise_backward.argtypes = [vp, vp, vp, vp, vp, i64, ci, vp]
        L.fsw_gating_grad_recompute.restype = ci
        L.fsw_gating_grad_recompute.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, vp]
        L.fsw_input_grad.restype = ci
        L.fsw_input_grad.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, i64, ci, vp]
        L.fsw_input_grad_noalloc.restype = ci
        L.fsw_input_grad_noalloc.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, vp]
        L.fsw_weight_grad.restype = ci
        L.fsw_weight_grad.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, i64, ci, vp]
        L.fsw_swiglu_backward.restype = ci
        L.fsw_swiglu_backward.argtypes = [vp] * 11 + [i64] * 7 + [vp, i64, ci, vp]
        for name in ("fsw_down_proj_forward", "fsw_down_proj_input_grad", "fsw_down_proj_weight_grad"):
            getattr(L, name).restype = ci
            getattr(L, name).argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, i64, ci, vp]
        L.fsw_workspace_bytes.restype = i64
        L.fsw_workspace_bytes.argtypes = [ci, i64, i64, i64]
        _lib = L
    return _lib


_bench_lib = None


def bench_lib() -> ctypes.CDLL:
    """The probe library of the benchmark harness (include/fusedswiglu_bench.h)."""
    global _bench_lib
    if _bench_lib is not None:
        return _bench_lib
    with _lock:
        if _bench_lib is None:
            if not os.path.exists(BENCH_LIBRARY_PATH):
                raise LibraryNotBuiltError(f"{BENCH_LIBRARY_PATH} not found; build it with `make -C {_CSRC}`")
            L = ctypes.CDLL(BENCH_LIBRARY_PATH)
            vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
            L.fsw_probe_mfma.restype = ci
            L.fsw_probe_mfma.argtypes = [ci, ci, ci, vp, vp, ctypes.POINTER(ctypes.c_double)]
            L.fsw_probe_stream_read.restype = ci
            L.fsw_probe_stream_read.argtypes = [vp, i64, vp, vp]
            L.fsw_probe_dma_read.argtypes = [vp, i64, ci, vp]
            L.fsw_probe_mfma_mix.restype = ci
            L.fsw_probe_mfma_mix.argtypes = [ci, ci, ci, vp, i64, vp, vp, ctypes.POINTER(ctypes.c_double)]
            _bench_lib = L
    return _bench_lib


def check(status: int) -> None:
    if status != 0:
        L = lib()
        msg = L.fsw_last_error().decode() or L.fsw_status_string(status).decode()
        raise FusedSwiGLUError(status, msg)
