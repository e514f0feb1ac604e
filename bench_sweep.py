#!/usr/bin/env python3
"""Sweep of the reference's published benchmark protocol on one MI355X.

The reference's README (README.md:41-63) plots TFLOP/s for batch 4, sequence 2048,
d_intermediate = 3 * d_model, d_model = 256 ... 4096, forward and forward+backward, bf16 and fp16,
for its fused kernels against eager PyTorch.  This script measures the same grid for this library
and for eager PyTorch (rocBLAS/hipBLASLt matmuls + elementwise kernels) on the same box and prints
a markdown table; with --out it also writes the table, the raw numbers (JSON) and the four plots of
the README (bf16 / fp16 x forward / forward+backward, fused against eager) into that directory.
Flop convention: forward 4*T*D*I, forward+backward 12*T*D*I.

    python bench_sweep.py [--step 128] [--iters 10] [--out DIR]
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
    ap.add_argument("--step", type=int, default=128, help="d_model step; 128 is the README's grid")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--out", default=None, help="directory for sweep.md, sweep.json and the four PNG plots")
    args = ap.parse_args()
    import torch

    from fusedswiglu_amd import FastAccumFusedSwiGLU, FusedSwiGLU

    dev = "cuda:0"
    B, S = 4, 2048
    T = B * S
    lines = ["| dtype | d_model | fused fwd TFLOP/s | eager fwd | fused fwd+bwd TFLOP/s | eager fwd+bwd |",
             "|---|---|---|---|---|---|"]
    print("\n".join(lines))
    rows = []
    for dtype, fn in ((torch.bfloat16, FusedSwiGLU), (torch.float16, FastAccumFusedSwiGLU)):
        for D in sorted(set([256] + list(range(256, 4097, args.step)) + [4096])):
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
            name = "bf16" if dtype == torch.bfloat16 else "fp16"
            lines.append(f"| {name} | {D} | {r[0]:.0f} | {r[1]:.0f} | {r[2]:.0f} | {r[3]:.0f} |")
            print(lines[-1], flush=True)
            rows.append({"dtype": name, "d_model": D, "fused_fwd": r[0], "eager_fwd": r[1], "fused_fwd_bwd": r[2], "eager_fwd_bwd": r[3]})
    if args.out:
        write_outputs(args.out, lines, rows, args.step)


def write_outputs(out_dir, lines, rows, step):
    import json

    import matplotlib

    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    os.makedirs(out_dir, exist_ok=True)
    head = (f"Sweep on the reference's published protocol (batch 4, sequence 2048, d_intermediate = 3 * d_model, "
            f"d_model 256 ... 4096 step {step}), one MI355X, `python bench_sweep.py --step {step} --out DIR`; "
            "TFLOP/s, fused = this library, eager = PyTorch matmuls + elementwise kernels on the same box.\n\n")
    with open(os.path.join(out_dir, "sweep.md"), "w") as f:
        f.write(head + "\n".join(lines) + "\n")
    with open(os.path.join(out_dir, "sweep.json"), "w") as f:
        json.dump(rows, f, indent=0)
    for name in ("bf16", "fp16"):
        sel = [r for r in rows if r["dtype"] == name]
        xs = [r["d_model"] for r in sel]
        for key, title in (("fwd", "forward"), ("fwd_bwd", "forward + backward")):
            plt.figure(figsize=(7, 4.2))
            plt.plot(xs, [r["fused_" + key] for r in sel], "o-", ms=3, label="fused (this library, MI355X)")
            plt.plot(xs, [r["eager_" + key] for r in sel], "s--", ms=3, label="eager PyTorch (rocBLAS/hipBLASLt)")
            plt.xlabel("d_model (batch 4, sequence 2048, d_intermediate = 3 d_model)")
            plt.ylabel("TFLOP/s")
            plt.title(f"SwiGLU {title}, {name}")
            plt.grid(alpha=0.3)
            plt.legend()
            plt.tight_layout()
            plt.savefig(os.path.join(out_dir, f"{name}_{key}.png"), dpi=110)
            plt.close()


if __name__ == "__main__":
    main()
