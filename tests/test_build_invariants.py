"""Properties of the compiled device code that the sources rely on but the compiler does not check (CPU only: the
kernels are cross-compiled to assembly, nothing runs).  The library's Makefile runs the same check on every build."""
import importlib.util
import os
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "flash-3-way-attention_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def _checker():
    spec = importlib.util.spec_from_file_location("check_m0", os.path.join(CSRC, "check_m0.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.check


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
@pytest.mark.parametrize("unit", ["tdp_bwd_mfma.hip", "dps_mfma.hip"])
def test_direct_lds_loads_own_m0(tmp_path, unit):
    """The direct-to-LDS loads set M0 in inline assembly; nothing the compiler emits in those kernels may use M0, and
    the LDS waits must stay counted (csrc/check_m0.py states the conditions)."""
    out = tmp_path / "unit.s"
    flags = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "--cuda-device-only", "-S"]
    subprocess.run([HIPCC, *flags, os.path.join(CSRC, unit), "-o", str(out)], check=True,
                   stderr=subprocess.DEVNULL, cwd=CSRC)
    assert _checker()(out.read_text()) is None


def test_checker_rejects_foreign_users_of_m0():
    check = _checker()
    ours = ("s_mov_b32 m0, s4\ns_nop 0\nglobal_load_lds_dwordx4 v1, s[2:3]\n" * 120 +
            "s_mov_b32 m0, s5\ns_nop 0\nglobal_load_lds_dword v2, s[2:3]\n" + "s_waitcnt lgkmcnt(4)\n")
    assert check(ours) is None
    assert "not ours" in check(ours + "s_movk_i32 m0, 0x100\n")
    assert "indirect" in check(ours + "s_set_gpr_idx_on s3, gpr_idx(SRC0)\n")
    assert "flushed" in check(ours.replace("lgkmcnt(4)", "lgkmcnt(0)"))
