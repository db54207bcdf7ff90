"""Properties of the compiled device code that the sources rely on but the compiler does not check (CPU only: the
kernels are cross-compiled to assembly, nothing runs)."""
import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flash-3-way-attention_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
def test_direct_lds_loads_own_m0(tmp_path):
    """`direct_load_16` is inline assembly that sets M0 (the LDS base of a direct-to-LDS load) without telling the
    compiler, which is sound only while nothing the compiler emits in those kernels uses M0: every reference to M0
    in the backward kernels' assembly must be one of ours, directly followed by its load, and no indirect register
    indexing (the compiler's own user of M0) may appear.  The LDS waits must also be counted, not flushed: the
    reason the loads are inline assembly at all."""
    out = tmp_path / "bwd.s"
    flags = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "--cuda-device-only", "-S"]
    subprocess.run([HIPCC, *flags, os.path.join(CSRC, "tdp_bwd_mfma.hip"), "-o", str(out)], check=True,
                   stderr=subprocess.DEVNULL, cwd=CSRC)
    lines = [ln.split(";")[0].strip() for ln in out.read_text().splitlines()]
    lines = [ln for ln in lines if ln and not ln.startswith(".")]
    uses = [i for i, ln in enumerate(lines) if re.search(r"\bm0\b", ln)]
    assert len(uses) > 100
    for i in uses:
        assert lines[i].startswith("s_mov_b32 m0,"), lines[i]
        assert lines[i + 1] == "s_nop 0" and lines[i + 2].startswith("global_load_lds_dwordx4"), lines[i:i + 3]
    text = "\n".join(lines)
    assert not re.search(r"s_set_gpr_idx|v_movrel|s_movrel", text)
    assert len([ln for ln in lines if ln.startswith("global_load_lds_dwordx4")]) == len(uses)
    # exact LDS wait counts in the kernels that keep stage loads in flight
    assert re.search(r"s_waitcnt lgkmcnt\((?:[4-9]|1[0-4])\)", text)
