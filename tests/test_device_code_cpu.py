"""A check of the generated gfx950 code (hipcc cross-compiles without a GPU).

Behind a `buffer_store_dwordx3/x4` whose scalar-offset operand is a REGISTER the compiler leaves out the wait state it
otherwise inserts before the next instruction that overwrites the store's data registers.  On MI355X that wait state is
needed: without it the tiled kernels' epilogue stored raw fp32 words of the following computation in a few lanes,
sporadically.  The kernels therefore put every offset of such a store into the vector operand; this test keeps it so."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "fusedswiglu_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-S", "--cuda-device-only", "-w"]


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
@pytest.mark.parametrize("source", ["fsw_tiled.hip", "fsw_skinny.hip", "fsw_generic.hip", "fsw_elementwise.hip"])
def test_wide_buffer_stores_carry_no_scalar_offset_register(source, tmp_path):
    out = tmp_path / (source + ".s")
    subprocess.run([HIPCC, *FLAGS, os.path.join(CSRC, source), "-o", str(out)], check=True, timeout=900)
    text = out.read_text()
    assert "v_mfma" in text or source == "fsw_elementwise.hip"          # really the device code
    stores = re.findall(r"^\s*buffer_store_dwordx[34]\s.*$", text, flags=re.M)
    risky = [s.strip() for s in stores if re.search(r",\s*s\d+\s+offen", s)]
    assert not risky, f"{len(risky)} wide buffer stores with a scalar offset register, e.g. {risky[0]}"
    if source == "fsw_tiled.hip":
        assert len(stores) > 100                                          # the epilogue's line stores are there
    # the compiled code keeps everything in registers (scratch would also change the launch requirements)
    spills = [int(n) for n in re.findall(r"\.vgpr_spill_count:\s+(\d+)", text)]
    assert spills and max(spills) == 0, f"register spills: {sorted(set(spills))}"
