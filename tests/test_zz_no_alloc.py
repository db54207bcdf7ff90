"""The allocation-free forward entry point (tritt_tdp_fwd_static_scratch) against tritt_tdp_fwd, through the
C ABI: same inputs, bitwise equal O and LSE, on calls in a row that share the library's static scratch."""
import ctypes
import math

import pytest
import torch

from flash_trittention import _lib

pytestmark = pytest.mark.gpu


def _both(B, H, T, D, dtype, windows=None, seed=0, poison=None):
    lib = _lib.lib()
    gen = torch.Generator(device="cpu").manual_seed(seed)
    ins = [torch.randn(B, H, T, D, generator=gen).to(dtype).cuda() for _ in range(5)]
    w = [T] * 4 if windows is None else list(windows)
    code = _lib.dtype_code(dtype)
    alpha = 1 / math.sqrt(D)
    stream = _lib.stream_ptr(ins[0].device)
    need = lib.tritt_tdp_fwd_workspace_bytes(B, H, T, D, code, 1, *w, 0)
    ws = _lib.workspace(need, ins[0].device)
    o_ref, lse_ref = torch.empty_like(ins[0]), torch.empty(B, H, T, device="cuda")
    rc = lib.tritt_tdp_fwd(*map(_lib.ptr, ins), _lib.ptr(o_ref), _lib.ptr(lse_ref), B, H, T, D, code, alpha, 1, *w,
                           _lib.ptr(ws), need, 0, stream)
    assert rc == 0, lib.tritt_status_string(rc)
    o = torch.full_like(ins[0], float("nan"))
    lse = torch.full((B, H, T), float("nan"), device="cuda")
    before = torch.cuda.memory_allocated()
    rc = lib.tritt_tdp_fwd_static_scratch(*map(_lib.ptr, ins), _lib.ptr(o), _lib.ptr(lse), B, H, T, D, code, alpha, 1,
                                          *w, 0, stream)
    assert rc == 0, lib.tritt_status_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(o, o_ref), f"O differs at B={B} H={H} T={T} D={D}"
    assert torch.equal(lse, lse_ref), f"LSE differs at B={B} H={H} T={T} D={D}"
    return o


def test_static_scratch_forward_matches_workspace_forward_on_consecutive_calls():
    print("static scratch: B=2 H=4 T=300 D=64 bf16, then B=1 H=2 T=100 D=64", flush=True)
    _both(2, 4, 300, 64, torch.bfloat16, seed=1)
    _both(1, 2, 100, 64, torch.bfloat16, seed=2)   # smaller: the scratch still holds the first call's data
    _both(1, 3, 33, 128, torch.float16, seed=3)
    _both(2, 2, 200, 64, torch.bfloat16, windows=(48, 64, 16, 24), seed=4)
    _both(1, 2, 64, 32, torch.float32, seed=5)     # fp32 VALU path: fp32 copies live in the scratch


def test_static_scratch_headline_shape_and_limit():
    lib = _lib.lib()
    assert lib.tritt_static_scratch_bytes() == 32 << 20
    _both(4, 8, 1024, 64, torch.bfloat16, seed=6)
    _both(1, 1, 128, 64, torch.bfloat16, seed=7)
    # a problem whose scratch exceeds the static array is refused before anything is launched
    one = ctypes.c_void_p(256)
    B, H, T, D = 8, 16, 4096, 128
    assert lib.tritt_tdp_fwd_workspace_bytes(B, H, T, D, _lib.TRITT_BF16, 1, T, T, T, T, 0) > (32 << 20)
    rc = lib.tritt_tdp_fwd_static_scratch(*[one] * 7, B, H, T, D, _lib.TRITT_BF16, 0.1, 1, T, T, T, T, 0, None)
    assert rc == -5
    assert b"static" in lib.tritt_status_string(rc)
