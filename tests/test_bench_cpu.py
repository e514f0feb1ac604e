"""CPU-side checks of the benchmark's bookkeeping: the HBM traffic it reports comes from the committed
counter profile, and that profile must belong to the kernel sources in the tree."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_traffic_is_parsed_from_the_committed_profile():
    traffic, stamp = bench.load_profiled_traffic()
    assert set(traffic) == {"forward_dual_gemm", "input_grad_dual_gemm", "weight_grad_dual_gemm"}
    T, D, I = 8192, 4096, 12288
    algorithmic = {  # bytes each kernel must move at least: operands once, results once
        "forward_dual_gemm": 2 * (T * D + 2 * D * I + 3 * T * I),
        "input_grad_dual_gemm": 2 * (2 * T * I + 2 * D * I + T * D),
        "weight_grad_dual_gemm": 2 * (T * D + 2 * T * I + 2 * D * I),
    }
    for name, measured in traffic.items():
        assert algorithmic[name] <= measured < 8 * algorithmic[name], (name, measured, algorithmic[name])
    assert stamp is not None and len(stamp) == 16


def test_profile_belongs_to_the_current_kernel_sources():
    """Fails when csrc/fsw_common.hpp, fsw_gemm.hpp or fsw_tiled.hip changed after the counter passes in
    profiles/gemm_kernels_c2_bf16.md were taken: re-run the passes named there and update the summary."""
    _, stamp = bench.load_profiled_traffic()
    assert stamp == bench.kernel_source_hash()


def test_parser_reads_the_table_format(tmp_path):
    text = ("| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | fetch scale | write scale |\n|---|---|---|---|---|\n"
            "| forward_dual_gemm | 1000 | 500 | 2.0 | 1.0 | x |\n| input_grad_dual_gemm | 10 | 5 | 1.5 | 1.0 |\n"
            "\nkernel-source-sha256: 0123456789abcdef (note)\n")
    p = tmp_path / "p.md"
    p.write_text(text)
    traffic, stamp = bench.load_profiled_traffic(str(p))
    assert traffic == {"forward_dual_gemm": 2500 * 1024, "input_grad_dual_gemm": 20 * 1024}
    assert stamp == "0123456789abcdef"
    assert bench.load_profiled_traffic(str(tmp_path / "missing.md")) == ({}, None)


def test_no_profiled_read_traffic_below_the_algorithmic_bytes():
    """Every row of the weight-streaming profile reads at least the bytes the launch must read (both weights and x
    once): a counter figure below that is an artefact of the summary (e.g. launches of different work averaged
    together), not a measurement, and must not be committed as traffic."""
    path = os.path.join(ROOT, "profiles", "skinny_forward_c4_bf16.md")
    rows = [l for l in open(path) if l.startswith("| fsw_") and "MiB" in l]
    assert len(rows) >= 8
    for l in rows:
        cells = [c.strip() for c in l.strip().strip("|").split("|")]
        scaled, requests, algorithmic = (float(c.split()[0]) for c in cells[2:5])
        assert scaled >= 0.995 * algorithmic and requests >= 0.995 * algorithmic, l
        assert scaled < 1.1 * algorithmic, l
