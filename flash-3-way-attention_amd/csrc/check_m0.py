"""Build check for translation units that include direct_lds.hpp.

`direct_load_16` and `direct_load_4` are inline assembly that writes M0 (the LDS base of a direct-to-LDS load).  M0 is a reserved
register: the compiler accepts it in a clobber list only with the note that it does not honour it, so the statement
is sound only while nothing the compiler emits in the same kernels uses M0.  This script reads the device assembly
of such a translation unit and fails unless every reference to M0 is one of ours (`s_mov_b32 m0` directly followed
by `s_nop 0` and its `global_load_lds_dwordx4` or `global_load_lds_dword`), no indirect register indexing (the compiler's own user of M0)
appears, and the waits for LDS reads in the kernels that keep stage loads in flight are counted rather than flushed
(the reason the loads are inline assembly at all).

usage: check_m0.py <file.s>      exit status 0 = sound
"""
import re
import sys


def check(text):
    lines = [ln.split(";")[0].strip() for ln in text.splitlines()]
    lines = [ln for ln in lines if ln and not ln.startswith(".")]
    uses = [i for i, ln in enumerate(lines) if re.search(r"\bm0\b", ln)]
    if len(uses) < 100:
        return "expected the direct loads of the kernels, found %d uses of m0" % len(uses)
    for i in uses:
        if not lines[i].startswith("s_mov_b32 m0,"):
            return "m0 used by an instruction that is not ours: " + lines[i]
        if lines[i + 1] != "s_nop 0" or not lines[i + 2].startswith("global_load_lds_dword"):
            return "m0 write not followed by its load: " + " | ".join(lines[i:i + 3])
    body = "\n".join(lines)
    if re.search(r"s_set_gpr_idx|v_movrel|s_movrel", body):
        return "indirect register indexing (a compiler-generated user of m0) present"
    if len([ln for ln in lines if ln.startswith("global_load_lds_dword")]) != len(uses):
        return "a direct-to-LDS load without its own m0 write"
    if not re.search(r"s_waitcnt lgkmcnt\((?:[4-9]|1[0-4])\)", body):
        return "no counted LDS wait left: the waits are being flushed to lgkmcnt(0)"
    return None


if __name__ == "__main__":
    problem = check(open(sys.argv[1]).read())
    if problem:
        sys.exit("check_m0: " + problem)
