"""The four calls into libtrittention_hip.so as functions of tensors, and the same four registered as
``torch.library`` custom ops (namespace ``flash_trittention``) with fake implementations.

Eager code calls the plain functions (no dispatcher overhead).  Under ``torch.compile`` the autograd Functions call
the custom ops instead, so tracing sees opaque ops with known output shapes instead of ctypes calls: the Functions
trace without graph breaks (``tests/test_gpu_compile.py``).  The C ABI stays the boundary; nothing here computes.
"""
from typing import List, Tuple

import torch

from . import _lib


def _empty_like_bhtd(q):
    return torch.empty(q.shape, dtype=q.dtype, device=q.device)


def _tdp_output(q, flags: int):
    """What tritt_tdp_fwd writes through `o`: one [B,H,T,D] tensor, or under FLAG_SPLIT_OPERANDS two of them
    stacked (the output and its rounding residual; the backward reads both)."""
    if flags & _lib.FLAG_SPLIT_OPERANDS:
        return torch.empty((2, *q.shape), dtype=q.dtype, device=q.device)
    return _empty_like_bhtd(q)


def tdp_fwd_impl(q, k1, k2, v1, v2, softmax_scale: float, causal: bool, k1_window: int, k2_window: int, kk_left: int,
                 kk_right: int, flags: int):
    _lib.require_gpu(q, "flash_trittention")
    q, k1, k2, v1, v2 = (_lib.view(t) for t in (q, k1, k2, v1, v2))
    lay = _lib.layouts((q, k1, k2, v1, v2))
    B, H, T, D = q.shape
    lib = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    o = _tdp_output(q, flags)
    lse = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
    shape = (B, H, T, D, code, float(softmax_scale), int(causal), k1_window, k2_window, kk_left, kk_right)
    with _lib.on_device(q.device):
        if lay is None:
            need = _lib.workspace_bytes("tritt_tdp_fwd_workspace_bytes", B, H, T, D, code, int(causal), k1_window,
                                        k2_window, kk_left, kk_right, flags)
            ws = _lib.workspace(need, q.device)
            st = lib.tritt_tdp_fwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(lse), *shape, _lib.ptr(ws), ws.numel(), flags, _lib.stream_ptr(q.device))
        else:  # strided views (a [B,T,H,D] projection output transposed, a slice of a fused tensor) are read in place
            need = _lib.workspace_bytes("tritt_tdp_fwd_strided_workspace_bytes", B, H, T, D, code, int(causal),
                                        k1_window, k2_window, kk_left, kk_right, flags, lay)
            ws = _lib.workspace(need, q.device)
            st = lib.tritt_tdp_fwd_strided(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), lay,
                                           _lib.ptr(o), _lib.ptr(lse), *shape, _lib.ptr(ws), ws.numel(), flags,
                                           _lib.stream_ptr(q.device))
    _lib.check(st, "tritt_tdp_fwd")
    return o, lse


def tdp_bwd_impl(q, k1, k2, v1, v2, o, lse, d_o, softmax_scale: float, causal: bool, k1_window: int, k2_window: int,
                 kk_left: int, kk_right: int, flags: int, wanted: int):
    """`wanted`: bit i set = gradient i of (dq, dk1, dk2, dv1, dv2) is computed; the others come back empty."""
    B, H, T, D = q.shape
    q, k1, k2, v1, v2, d_o = (_lib.view(t) for t in (q, k1, k2, v1, v2, d_o))
    lay, lay_do = _lib.layouts((q, k1, k2, v1, v2)), _lib.layouts((d_o,))
    lib = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    grads = [_empty_like_bhtd(q) if (wanted >> i) & 1 else None for i in range(5)]
    gptr = [_lib.ptr(t) if t is not None else None for t in grads]
    shape = (B, H, T, D, code, float(softmax_scale), int(causal), k1_window, k2_window, kk_left, kk_right)
    with _lib.on_device(q.device):
        if lay is None and lay_do is None:
            need = _lib.workspace_bytes("tritt_tdp_bwd_workspace_bytes", B, H, T, D, code, int(causal), k1_window,
                                        k2_window, kk_left, kk_right, flags)
            ws = _lib.workspace(need, q.device)
            st = lib.tritt_tdp_bwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(lse), _lib.ptr(d_o), *gptr, *shape, _lib.ptr(ws), ws.numel(), flags,
                                   _lib.stream_ptr(q.device))
        else:
            need = _lib.workspace_bytes("tritt_tdp_bwd_strided_workspace_bytes", B, H, T, D, code, int(causal),
                                        k1_window, k2_window, kk_left, kk_right, flags, lay, lay_do)
            ws = _lib.workspace(need, q.device)
            st = lib.tritt_tdp_bwd_strided(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), lay,
                                           _lib.ptr(o), _lib.ptr(lse), _lib.ptr(d_o), lay_do, *gptr, *shape,
                                           _lib.ptr(ws), ws.numel(), flags, _lib.stream_ptr(q.device))
    _lib.check(st, "tritt_tdp_bwd")
    return grads


def dps_fwd_impl(q, k1, k2, v1, v2, softmax_scale: float, causal: bool, k_diff: int, flags: int):
    _lib.require_gpu(q, "TrittentionTriton")
    q, k1, k2, v1, v2 = (_lib.view(t) for t in (q, k1, k2, v1, v2))
    lay = _lib.layouts((q, k1, k2, v1, v2))
    B, H, T, D = q.shape
    lib = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    o = _empty_like_bhtd(q)
    m = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
    shape = (B, H, T, D, code, float(softmax_scale), int(causal), k_diff)
    with _lib.on_device(q.device):
        if lay is None:
            ws = _lib.workspace(_lib.workspace_bytes("tritt_dps_fwd_workspace_bytes", B, H, T, D, code, flags), q.device)
            st = lib.tritt_dps_fwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(m), *shape, _lib.ptr(ws), ws.numel(), flags, _lib.stream_ptr(q.device))
        else:
            ws = _lib.workspace(_lib.workspace_bytes("tritt_dps_fwd_strided_workspace_bytes", B, H, T, D, code, flags,
                                                     lay), q.device)
            st = lib.tritt_dps_fwd_strided(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), lay,
                                           _lib.ptr(o), _lib.ptr(m), *shape, _lib.ptr(ws), ws.numel(), flags,
                                           _lib.stream_ptr(q.device))
    _lib.check(st, "tritt_dps_fwd")
    return o, m


def dps_bwd_impl(q, k1, k2, v1, v2, o, m, d_o, softmax_scale: float, causal: bool, k_diff: int, flags: int):
    B, H, T, D = q.shape
    q, k1, k2, v1, v2, d_o = (_lib.view(t) for t in (q, k1, k2, v1, v2, d_o))
    lay, lay_do = _lib.layouts((q, k1, k2, v1, v2)), _lib.layouts((d_o,))
    lib = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    grads = [_empty_like_bhtd(q) for _ in range(5)]
    gptr = [_lib.ptr(t) for t in grads]
    shape = (B, H, T, D, code, float(softmax_scale), int(causal), k_diff)
    with _lib.on_device(q.device):
        if lay is None and lay_do is None:
            ws = _lib.workspace(_lib.workspace_bytes("tritt_dps_bwd_workspace_bytes", B, H, T, D, code, flags), q.device)
            st = lib.tritt_dps_bwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(m), _lib.ptr(d_o), *gptr, *shape, _lib.ptr(ws), ws.numel(), flags,
                                   _lib.stream_ptr(q.device))
        else:
            ws = _lib.workspace(_lib.workspace_bytes("tritt_dps_bwd_strided_workspace_bytes", B, H, T, D, code, flags,
                                                     lay, lay_do), q.device)
            st = lib.tritt_dps_bwd_strided(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), lay,
                                           _lib.ptr(o), _lib.ptr(m), _lib.ptr(d_o), lay_do, *gptr, *shape, _lib.ptr(ws),
                                           ws.numel(), flags, _lib.stream_ptr(q.device))
    _lib.check(st, "tritt_dps_bwd")
    return grads


# ---------------------------------------------------------------- torch.library registration (used under torch.compile)
_T = torch.Tensor


@torch.library.custom_op("flash_trittention::tdp_fwd", mutates_args=())
def tdp_fwd_op(q: _T, k1: _T, k2: _T, v1: _T, v2: _T, softmax_scale: float, causal: bool, k1_window: int,
               k2_window: int, kk_left: int, kk_right: int, flags: int) -> Tuple[_T, _T]:
    return tdp_fwd_impl(q, k1, k2, v1, v2, softmax_scale, causal, k1_window, k2_window, kk_left, kk_right, flags)


@tdp_fwd_op.register_fake
def _(q, k1, k2, v1, v2, softmax_scale, causal, k1_window, k2_window, kk_left, kk_right, flags):
    return _tdp_output(q, flags), q.new_empty(q.shape[:3], dtype=torch.float32)


@torch.library.custom_op("flash_trittention::tdp_bwd", mutates_args=())
def tdp_bwd_op(q: _T, k1: _T, k2: _T, v1: _T, v2: _T, o: _T, lse: _T, d_o: _T, softmax_scale: float, causal: bool,
               k1_window: int, k2_window: int, kk_left: int, kk_right: int, flags: int, wanted: int) -> List[_T]:
    grads = tdp_bwd_impl(q, k1, k2, v1, v2, o, lse, d_o, softmax_scale, causal, k1_window, k2_window, kk_left,
                         kk_right, flags, wanted)
    return [g if g is not None else q.new_empty(0) for g in grads]


@tdp_bwd_op.register_fake
def _(q, k1, k2, v1, v2, o, lse, d_o, softmax_scale, causal, k1_window, k2_window, kk_left, kk_right, flags, wanted):
    return [_empty_like_bhtd(q) if (wanted >> i) & 1 else q.new_empty(0) for i in range(5)]


@torch.library.custom_op("flash_trittention::dps_fwd", mutates_args=())
def dps_fwd_op(q: _T, k1: _T, k2: _T, v1: _T, v2: _T, softmax_scale: float, causal: bool, k_diff: int,
               flags: int) -> Tuple[_T, _T]:
    return dps_fwd_impl(q, k1, k2, v1, v2, softmax_scale, causal, k_diff, flags)


@dps_fwd_op.register_fake
def _(q, k1, k2, v1, v2, softmax_scale, causal, k_diff, flags):
    return _empty_like_bhtd(q), q.new_empty(q.shape[:3], dtype=torch.float32)


@torch.library.custom_op("flash_trittention::dps_bwd", mutates_args=())
def dps_bwd_op(q: _T, k1: _T, k2: _T, v1: _T, v2: _T, o: _T, m: _T, d_o: _T, softmax_scale: float, causal: bool,
               k_diff: int, flags: int) -> List[_T]:
    return dps_bwd_impl(q, k1, k2, v1, v2, o, m, d_o, softmax_scale, causal, k_diff, flags)


@dps_bwd_op.register_fake
def _(q, k1, k2, v1, v2, o, m, d_o, softmax_scale, causal, k_diff, flags):
    return [_empty_like_bhtd(q) for _ in range(5)]


def compiling() -> bool:
    return torch.compiler.is_compiling()
