#!/usr/bin/env python3
"""Benchmark of the fused SwiGLU forward+backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one `FusedSwiGLU.apply(x, Wg, Wu)` forward plus `out.backward(dout)` on synthetic,
HBM-resident bf16 inputs of the headline configuration (x [4,2048,4096], Wg/Wu [4096,12288],
all ~N(0,1) resp. N(0,1/D), seed 0).  Prints ONE JSON line: whole-step TFLOP/s (12*T*D*I flop per
step), a roofline object for the dominant kernel measured live with GPU events on the launch
stream, and the eager fp32 PyTorch SwiGLU timed on this machine's host cores as CPU baseline.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM-side bytes per launch (L2 <-> fabric reads + writes) of the three GEMM kernels at the C2 shape come
# from the FETCH_SIZE / WRITE_SIZE counter passes summarised in this file (bench.py cannot run the profiler
# itself).  The summary is stamped with a hash of the kernel sources it was taken with; when the sources
# have changed since, `traffic` is reported as null instead of a stale figure.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_kernels_c2_bf16.md")
KERNEL_SOURCES = ("fsw_common.hpp", "fsw_gemm.hpp", "fsw_gemm4.hpp", "fsw_tiled.hip")


def kernel_source_hash():
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "fusedswiglu_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def load_profiled_traffic(path=TRAFFIC_PROFILE):
    """({kernel: HBM bytes per launch}, source hash the profile was taken with) parsed from the table
    `| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | fetch scale | write scale |` of the profile summary."""
    import re

    traffic, stamp = {}, None
    try:
        text = open(path).read()
    except OSError:
        return traffic, stamp
    for m in re.finditer(r"^\|\s*(\w+_dual_gemm)\s*\|\s*(\d+)\s*\|\s*(\d+)\s*\|\s*([\d.]+)\s*\|\s*([\d.]+)\s*\|", text, flags=re.M):
        name, fetch, write, fs, ws = m.group(1), int(m.group(2)), int(m.group(3)), float(m.group(4)), float(m.group(5))
        traffic[name] = int((fetch * fs + write * ws) * 1024)
    m = re.search(r"kernel-source-sha256:\s*([0-9a-f]{16})", text)
    if m:
        stamp = m.group(1)
    return traffic, stamp


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the skinny-M and per-kernel extras")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run launches of known HBM traffic (1 GiB plain copies, streaming reads and "
                         "direct-to-LDS reads) so that profiler byte counters collected over this run can be scaled")
    return ap.parse_args()


def gpu_time_ms(fn, iters, warmup=3):
    """Average GPU duration of fn() over `iters` back-to-back launches, from events recorded on
    the stream the kernels are launched on (torch's current stream)."""
    import torch

    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def other_configs(dev, c2_tensors):
    """Event-timed fwd+bwd steps beside the headline: C3 (fp16, ragged I) and C5 (bf16, large) fused and
    eager, the eager step and the memory-saving (recompute) step at C2, and single vendor GEMMs of the
    three operand layouts at the C2 shape.  TFLOP/s by the same convention (12*T*D*I per step)."""
    import torch
    import torch.nn.functional as F

    from fusedswiglu_amd import FastAccumFusedSwiGLU, FusedSwiGLU
    from fusedswiglu_amd.ops import swiglu

    def fused_step(fn, x, wg, wu, dout):
        def run():
            x.grad = wg.grad = wu.grad = None
            fn(x, wg, wu).backward(dout)
        return run

    def eager_step(x, wg, wu, dout):
        def run():
            x.grad = wg.grad = wu.grad = None
            (F.silu(x @ wg) * (x @ wu)).backward(dout)
        return run

    def rec(ms, flop):
        return {"ms": round(ms, 4), "tflops": round(flop / ms / 1e9, 1)}

    out = {}
    x, wg, wu, dout = c2_tensors
    T, D, I = x.shape[0] * x.shape[1], x.shape[2], wg.shape[1]
    flop = 12.0 * T * D * I
    out["C2_bf16"] = {
        "shape": "x [4,2048,4096], W [4096,12288]",
        "fused": rec(gpu_time_ms(fused_step(FusedSwiGLU.apply, x, wg, wu, dout), iters=10), flop),
        "fused_recompute": rec(gpu_time_ms(fused_step(lambda a, b, c: swiglu(a, b, c, recompute=True), x, wg, wu, dout), iters=10), flop),
        "eager_pytorch": rec(gpu_time_ms(eager_step(x, wg, wu, dout), iters=10), flop),
    }
    # single vendor GEMMs (torch.matmul -> hipBLASLt/rocBLAS) of the three layouts, 2*T*D*I flop each
    xd, wd = x.detach().reshape(T, D), wg.detach()
    dg = dout.reshape(T, I)
    gflop = 2.0 * T * D * I
    out["C2_bf16"]["vendor_gemm"] = {
        "NN_forward_like": rec(gpu_time_ms(lambda: torch.matmul(xd, wd), iters=10), gflop),
        "NT_input_grad_like": rec(gpu_time_ms(lambda: torch.matmul(dg, wd.t()), iters=10), gflop),
        "TN_weight_grad_like": rec(gpu_time_ms(lambda: torch.matmul(xd.t(), dg), iters=10), gflop),
    }
    for name, fn, dt, xs, I2, iters in (("C3_fp16", FastAccumFusedSwiGLU.apply, torch.float16, (2, 4096, 4096), 11008, 10),
                                        ("C5_bf16", FusedSwiGLU.apply, torch.bfloat16, (8, 4096, 8192), 28672, 3)):
        torch.manual_seed(1)
        D2 = xs[-1]
        x2 = torch.randn(*xs, device=dev, dtype=torch.float32).to(dt).requires_grad_(True)
        wg2 = (torch.randn(D2, I2, device=dev, dtype=torch.float32) / D2 ** 0.5).to(dt).requires_grad_(True)
        wu2 = (torch.randn(D2, I2, device=dev, dtype=torch.float32) / D2 ** 0.5).to(dt).requires_grad_(True)
        dy2 = torch.randn(*xs[:-1], I2, device=dev, dtype=torch.float32).to(dt)
        fl2 = 12.0 * xs[0] * xs[1] * D2 * I2
        out[name] = {
            "shape": f"x {list(xs)}, W [{D2},{I2}]",
            "fused": rec(gpu_time_ms(fused_step(fn, x2, wg2, wu2, dy2), iters=iters, warmup=2), fl2),
            "eager_pytorch": rec(gpu_time_ms(eager_step(x2, wg2, wu2, dy2), iters=iters, warmup=2), fl2),
        }
        out[name]["fused_over_eager"] = round(out[name]["eager_pytorch"]["ms"] / out[name]["fused"]["ms"], 3)
        del x2, wg2, wu2, dy2
        torch.cuda.empty_cache()
    out["C2_bf16"]["fused_over_eager"] = round(out["C2_bf16"]["eager_pytorch"]["ms"] / out["C2_bf16"]["fused"]["ms"], 3)
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no collective, sharding or rank code "
              "is part of it, so there is no figure at several GPUs to report)", file=sys.stderr)
        sys.exit(2)

    import torch

    from fusedswiglu_amd import FusedSwiGLU, _abi

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    L = _abi.lib()  # raises if the HIP library is not built: no fallback
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    dt = torch.bfloat16
    B, S, D, I = 4, 2048, 4096, 12288
    T = B * S
    x = torch.randn(B, S, D, device=dev, dtype=torch.float32).to(dt).requires_grad_(True)
    wg = (torch.randn(D, I, device=dev, dtype=torch.float32) / D ** 0.5).to(dt).requires_grad_(True)
    wu = (torch.randn(D, I, device=dev, dtype=torch.float32) / D ** 0.5).to(dt).requires_grad_(True)
    dout = torch.randn(B, S, I, device=dev, dtype=torch.float32).to(dt)

    def step():
        x.grad = wg.grad = wu.grad = None
        out = FusedSwiGLU.apply(x, wg, wu)
        out.backward(dout)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms_per_step = dt_s * 1e3 / args.steps
    flop_step = 12.0 * T * D * I
    tflops = flop_step / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel durations through the C ABI (pre-allocated buffers, launch stream events)
    stream = torch.cuda.current_stream(dev).cuda_stream
    xd, wgd, wud = x.detach(), wg.detach(), wu.detach()
    out = torch.empty(B, S, I, device=dev, dtype=dt)
    g, u = torch.empty_like(out), torch.empty_like(out)
    dG, dU = torch.empty_like(out), torch.empty_like(out)
    dx = torch.empty(B, S, D, device=dev, dtype=dt)
    dWg, dWu = torch.empty(D, I, device=dev, dtype=dt), torch.empty(D, I, device=dev, dtype=dt)
    p = lambda t: t.data_ptr()  # noqa: E731
    calls = {
        "forward_dual_gemm": (lambda: _abi.check(L.fsw_swiglu_forward(p(xd), p(wgd), p(wud), p(out), p(g), p(u), T, D, I, D, I, I, 0, stream)), 4.0 * T * D * I),
        "elementwise_backward": (lambda: _abi.check(L.fsw_elementwise_backward(p(dout), p(g), p(u), p(dU), p(dG), T * I, 0, stream)), None),
        "input_grad_dual_gemm": (lambda: _abi.check(L.fsw_input_grad(p(dG), p(dU), p(wgd), p(wud), p(dx), T, D, I, I, I, D, None, 0, 0, stream)), 4.0 * T * D * I),
        "weight_grad_dual_gemm": (lambda: _abi.check(L.fsw_weight_grad(p(xd), p(dU), p(dG), p(dWu), p(dWg), T, D, I, D, I, I, None, 0, 0, stream)), 4.0 * T * D * I),
    }
    kernels = {}
    for name, (fn, flop) in calls.items():
        ms = gpu_time_ms(fn, iters=max(5, args.steps))
        rec = {"ms": round(ms, 4)}
        if flop is not None:
            rec["tflops"] = round(flop / ms / 1e9, 1)
            rec["frac_mfma_peak"] = round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4)
        else:
            rec["gbs"] = round(10.0 * T * I / ms / 1e6, 1)  # 3 reads + 2 writes of 2 bytes per element
            rec["frac_hbm_peak"] = round(rec["gbs"] / PEAK_HBM_GBS, 4)
        kernels[name] = rec
    profiled, stamp = load_profiled_traffic()
    gemm_names = [k for k in kernels if "tflops" in kernels[k]]
    dominant = max(gemm_names, key=lambda k: kernels[k]["ms"])
    achieved = 4.0 * T * D * I / kernels[dominant]["ms"] / 1e9
    roofline = {
        "kernel": dominant,
        "bound": "mfma",
        "achieved": round(achieved, 1),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
        "traffic": profiled.get(dominant) if stamp == kernel_source_hash() else None,
        "algorithmic_flop_per_launch": 4.0 * T * D * I,
    }
    if roofline["traffic"] is None:
        roofline["traffic_note"] = "no counter profile of the current kernel sources in profiles/gemm_kernels_c2_bf16.md"

    result = {
        "metric": "fwd+bwd TFLOP/s & % bf16 MFMA peak, 8192 tok, d=4096->12288",
        "value": round(tflops, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "C2: bf16 FusedSwiGLU fwd+bwd, x [4,2048,4096], Wg/Wu [4096,12288], "
                               "dout ~ N(0,1), fp32 MFMA accumulate", "tokens": T, "d_model": D,
                   "d_intermediate": I, "flop_per_step": flop_step},
        "pct_of_bf16_mfma_peak": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
        "roofline": roofline,
        "kernels": kernels,
    }

    # ---- practical ceilings of this machine: register-only MFMA loop and a streaming read
    if not args.no_extra:
        sink = torch.zeros(4, device=dev, dtype=torch.float32)
        ncu = torch.cuda.get_device_properties(dev).multi_processor_count
        ceil = {}
        for name, rnd in (("mfma_constant_operands_tflops", 0), ("mfma_normal_operands_tflops", 1)):
            fl = ctypes.c_double(0.0)
            run = lambda: _abi.check(_abi.bench_lib().fsw_probe_mfma(rnd, 20000, ncu, p(sink), stream, ctypes.byref(fl)))  # noqa: E731
            ms = gpu_time_ms(run, iters=3, warmup=1)
            ceil[name] = round(fl.value / ms / 1e9, 1)
        # the 16x16x32 instruction the tiled kernels use (mix 0 of the probe: no data movement beside it)
        window = torch.empty(8 << 20, device=dev, dtype=torch.uint8).fill_(60)
        # mix 1: the tiled kernels' LDS reads and direct loads beside the MFMAs; mix 5: the same with the
        # weight-side fragments formed by the gating-gradient arithmetic instead of held in registers - what the
        # matrix cores would deliver to a weight-gradient GEMM that absorbed the gating-gradient kernel
        for name, mix in (("mfma_16x16x32_normal_operands_tflops", 0),
                          ("mfma_16x16x32_with_tile_data_movement_tflops", 1),
                          ("mfma_16x16x32_with_gating_gradient_in_operand_path_tflops", 5)):
            fl = ctypes.c_double(0.0)
            run = lambda: _abi.check(_abi.bench_lib().fsw_probe_mfma_mix(mix, 10000, 2 * ncu, p(window), window.numel(), p(sink), stream, ctypes.byref(fl)))  # noqa: E731
            ms = gpu_time_ms(run, iters=3, warmup=1)
            ceil[name] = round(fl.value / ms / 1e9, 1)
        del window
        big = torch.empty(1 << 31, device=dev, dtype=torch.uint8).fill_(1)
        ms = gpu_time_ms(lambda: _abi.check(_abi.bench_lib().fsw_probe_stream_read(p(big), big.numel(), p(sink), stream)), iters=5, warmup=2)
        # the rate of a plain streaming-read kernel, for orientation: not a bound (the weight-streaming kernels
        # and the elementwise kernel may exceed it)
        ceil["hbm_read_probe_gbs"] = round(big.numel() / ms / 1e6, 1)
        del big
        result["measured_ceilings"] = ceil

    if args.calibrate_copy:
        # launches of known HBM traffic (1 GiB each, far beyond the caches), three of each: a plain copy, a
        # streaming read, and the kernels' own request pattern (direct global->LDS loads of whole lines, without
        # and with the non-temporal hint)
        src = torch.empty(1 << 30, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty_like(src)
        sink = torch.zeros(4, device=dev, dtype=torch.float32)
        B = _abi.bench_lib()
        for _ in range(3):
            dst.copy_(src)
            _abi.check(B.fsw_probe_stream_read(p(dst), dst.numel(), p(sink), stream))
            _abi.check(B.fsw_probe_dma_read(p(src), src.numel(), 0, stream))
            _abi.check(B.fsw_probe_dma_read(p(dst), dst.numel(), 1, stream))
        torch.cuda.synchronize()
        del src, dst

    # ---- skinny-M forward (weight streaming, HBM bound), forward only, no pre-activation stores
    if not args.no_extra:
        D4, I4 = 8192, 28672
        w_sets = [((torch.randn(D4, I4, device=dev, dtype=dt) / D4 ** 0.5), (torch.randn(D4, I4, device=dev, dtype=dt) / D4 ** 0.5))
                  for _ in range(2)]

        def stream_runs(sets, flag, ldw):
            runs = []
            for M in (16, 64, 128, 256):
                xs = torch.randn(M, D4, device=dev, dtype=dt)
                os_ = torch.empty(M, I4, device=dev, dtype=dt)
                state = {"i": 0}

                def fwd():
                    a, b = sets[state["i"] & 1]  # alternate weight sets: nothing stays cache resident
                    state["i"] += 1
                    _abi.check(L.fsw_swiglu_forward(p(xs), p(a), p(b), p(os_), None, None, M, D4, I4, D4, ldw, I4, flag, stream))

                ms = gpu_time_ms(fwd, iters=20)
                nbytes = 2.0 * (2 * D4 * I4 + M * D4 + M * I4)
                runs.append({"M": M, "ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
                             "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                             "tflops": round(4.0 * M * D4 * I4 / ms / 1e9, 1)})
            return runs

        skinny = stream_runs(w_sets, 0, I4)
        # the same weights viewed as [I, D] storage (the values do not matter for the timing)
        skinny_out_in = stream_runs([(a.view(I4, D4), b.view(I4, D4)) for a, b in w_sets], _abi.WEIGHTS_OUT_IN, D4)
        result["skinny_forward"] = {"workload": "C4: bf16 forward, x [M,8192], Wg/Wu [8192,28672]", "bound": "hbm",
                                    "peak_gbs": PEAK_HBM_GBS, "runs": skinny,
                                    "workload_weights_out_in": "the same with Wg/Wu stored [28672,8192] (nn.Linear layout)",
                                    "runs_weights_out_in": skinny_out_in}
        # the down projection that follows, same model (y [M,8192] = act [M,28672] W_down), both storage orders
        def down_runs(w_list, flag, ldw):
            runs = []
            scratch = torch.empty(int(L.fsw_workspace_bytes(_abi.STEP_DOWN_FORWARD | flag, 128, D4, I4)) or 16, device=dev, dtype=torch.uint8)
            for M in (16, 64, 128):
                act = torch.randn(M, I4, device=dev, dtype=dt)
                y = torch.empty(M, D4, device=dev, dtype=dt)
                state = {"i": 0}

                def down():
                    w = w_list[state["i"] % len(w_list)]
                    state["i"] += 1
                    _abi.check(L.fsw_down_proj_forward(p(act), p(w), p(y), M, I4, D4, I4, ldw, D4, p(scratch), scratch.numel(), flag, stream))

                def vendor():
                    w = w_list[state["i"] % len(w_list)]
                    state["i"] += 1
                    torch.matmul(act, w.t() if flag else w, out=y)

                ms, ms_v = gpu_time_ms(down, iters=20), gpu_time_ms(vendor, iters=20)
                nbytes = 2.0 * (D4 * I4 + M * I4 + M * D4)
                runs.append({"M": M, "ms": round(ms, 4), "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                             "vendor_ms": round(ms_v, 4), "vendor_frac_hbm_peak": round(nbytes / ms_v / 1e6 / PEAK_HBM_GBS, 4)})
            return runs

        flat = [w for pair in w_sets for w in pair]   # four arrays of D4*I4 elements, alternating: nothing stays cached
        result["down_proj_few_tokens"] = {
            "workload": "bf16 y [M,8192] = act [M,28672] W_down, W_down read once; vendor = torch.matmul on the same arrays",
            "runs_w_down_DxI": down_runs([w.view(D4, I4) for w in flat], _abi.WEIGHTS_OUT_IN, I4),
            "runs_w_down_IxD": down_runs([w.view(I4, D4) for w in flat], 0, D4)}
        del w_sets, flat

    # ---- the other configurations, the eager PyTorch step and the vendor GEMMs on the same box
    if not args.no_extra:
        del out, g, u, dG, dU, dx, dWg, dWu
        result["other_configs"] = other_configs(dev, (x, wg, wu, dout))

    # ---- CPU baseline: the eager fp32 SwiGLU of the reference's test on this machine's host cores
    if not args.no_cpu_baseline:
        from oracle import swiglu_oracle as osw

        torch.manual_seed(0)
        Bc, Sc, Dc, Ic = 4, 2048, 1024, 3072
        xc = torch.randn(Bc, Sc, Dc)
        wgc, wuc = torch.randn(Dc, Ic) / Dc ** 0.5, torch.randn(Dc, Ic) / Dc ** 0.5
        dyc = torch.randn(Bc, Sc, Ic)
        osw.eager_torch_fwd_bwd(xc, wgc, wuc, dyc)  # warm-up
        best = float("inf")
        t_all = time.perf_counter()
        reps = 0
        while reps < 3 or (time.perf_counter() - t_all < 10.0 and reps < 30):
            t1 = time.perf_counter()
            osw.eager_torch_fwd_bwd(xc, wgc, wuc, dyc)
            best = min(best, time.perf_counter() - t1)
            reps += 1
        fl = 12.0 * Bc * Sc * Dc * Ic
        result["cpu_baseline"] = {
            "value": round(fl / best / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"C1: eager fp32 PyTorch SwiGLU fwd+bwd, x [4,2048,1024], W [1024,3072]; best of {reps} "
                      f"after a warm-up, {best * 1e3:.1f} ms; os.cpu_count()={os.cpu_count()}",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
