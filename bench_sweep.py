#!/usr/bin/env python3
"""Sweep of the reference's published benchmark protocol on one MI355X.

The reference's README (README.md:41-63) plots TFLOP/s for batch 4, sequence 2048,
d_intermediate = 3 * d_model, d_model = 256 ... 4096, forward and forward+backward, bf16 and fp16,
for its fused kernels against eager PyTorch.  This script measures the same grid for this library
and for eager PyTorch (rocBLAS/hipBLASLt matmuls + elementwise kernels) on the same box and prints
a markdown table.  Flop convention: forward 4*T*D*I, forward+backward 12*T*D*I.

    python bench_sweep.py [--step 512] [--iters 10]
"""
import argparse
import sys
import os

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def time_ms(fn, iters, warmup=3, min_ms=40.0):
    """Mean time per call: `iters` calls, repeated until the timed region is at least `min_ms` long
    (the small shapes of the sweep run a few microseconds per call)."""
    import torch

    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while True:
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        e1.synchronize()
        total = e0.elapsed_time(e1)
        if total >= min_ms or iters >= 100000:
            return total / iters
        iters = int(iters * max(2.0, 1.2 * min_ms / max(total, 1e-3)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--step", type=int, default=512)
    ap.add_argument("--iters", type=int, default=10)
    args = ap.parse_args()
    import torch

    from fusedswiglu_amd import FastAccumFusedSwiGLU, FusedSwiGLU

    dev = "cuda:0"
    B, S = 4, 2048
    T = B * S
    print("| dtype | d_model | fused fwd TFLOP/s | eager fwd | fused fwd+bwd TFLOP/s | eager fwd+bwd |")
    print("|---|---|---|---|---|---|")
    for dtype, fn in ((torch.bfloat16, FusedSwiGLU), (torch.float16, FastAccumFusedSwiGLU)):
        for D in [256] + list(range(args.step, 4097, args.step)):
            I = 3 * D
            torch.manual_seed(0)
            x = torch.randn(B, S, D, device=dev, dtype=dtype, requires_grad=True)
            wg = (torch.randn(D, I, device=dev, dtype=torch.float32) / D ** 0.5).to(dtype).requires_grad_(True)
            wu = (torch.randn(D, I, device=dev, dtype=torch.float32) / D ** 0.5).to(dtype).requires_grad_(True)
            dy = torch.randn(B, S, I, device=dev, dtype=dtype)

            def eager_fwd():
                with torch.no_grad():
                    return torch.nn.functional.silu(x @ wg) * (x @ wu)

            def fused_fwd():
                with torch.no_grad():
                    return fn.apply(x, wg, wu)

            def eager_fb():
                x.grad = wg.grad = wu.grad = None
                (torch.nn.functional.silu(x @ wg) * (x @ wu)).backward(dy)

            def fused_fb():
                x.grad = wg.grad = wu.grad = None
                fn.apply(x, wg, wu).backward(dy)

            f = 4.0 * T * D * I
            r = [f / time_ms(fused_fwd, args.iters) / 1e9, f / time_ms(eager_fwd, args.iters) / 1e9,
                 3 * f / time_ms(fused_fb, args.iters) / 1e9, 3 * f / time_ms(eager_fb, args.iters) / 1e9]
            print(f"| {'bf16' if dtype == torch.bfloat16 else 'fp16'} | {D} | {r[0]:.0f} | {r[1]:.0f} | {r[2]:.0f} | {r[3]:.0f} |", flush=True)


if __name__ == "__main__":
    main()
