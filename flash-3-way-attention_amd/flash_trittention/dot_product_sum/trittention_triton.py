"""Dot-product-sum trittention on MI355X.

Mirrors ``TrittentionTritonFunction`` / ``TrittentionTriton`` of the reference
(dot_product_sum/trittention_triton.py:15-125 forward, :127-359 backward,
:362-403 module).  The class names are kept so existing imports keep working;
the kernels underneath are HIP, evaluated as two chained attention passes.
The module returns ``(o, m)`` with ``m`` the per-row logsumexp, like the
reference.
"""
from typing import Optional

import torch
import torch.nn as nn

from .. import _lib
from ..triple_dot_product.utils import clamp_window


class TrittentionTritonFunction(torch.autograd.Function):
    # `flags` of the C ABI; a class constant (see FlashTrittention.IMPL_FLAGS)
    IMPL_FLAGS = _lib.FLAG_AUTO

    @classmethod
    def with_flags(cls, flags: int):
        return _lib.flagged_subclass(cls, flags)

    @staticmethod
    def forward(ctx, q, k1, k2, v1, v2, causal, softmax_scale, k_diff, convert_to_float32=False,
                input_precision=None):
        if not (q.shape == k1.shape == k2.shape == v1.shape == v2.shape):
            raise ValueError(f"Shape mismatch: q={q.shape}, k1={k1.shape}, k2={k2.shape}, v1={v1.shape}, "
                             f"v2={v2.shape}")
        if not (q.dtype == k1.dtype == k2.dtype == v1.dtype == v2.dtype):
            raise ValueError("q, k1, k2, v1, v2 must all have the same dtype")
        if not (q.device == k1.device == k2.device == v1.device == v2.device):
            raise ValueError("q, k1, k2, v1, v2 must all be on the same device")
        if q.dim() != 4:
            raise ValueError(f"expected [batch, heads, seq_len, head_dim] tensors, got shape {tuple(q.shape)}")
        B, H, T, D = q.shape
        if D not in (16, 32, 64, 128):
            raise ValueError(f"head_dim must be one of 16, 32, 64, 128, got {D}")
        code = _lib.dtype_code(q.dtype)
        _lib.require_gpu(q, "TrittentionTriton")
        q, k1, k2, v1, v2 = (_lib.dense(t) for t in (q, k1, k2, v1, v2))
        k_diff = clamp_window(k_diff, T, "k_diff")
        flags = getattr(getattr(ctx, "_forward_cls", None), "IMPL_FLAGS", _lib.FLAG_AUTO)
        if convert_to_float32 and not flags & _lib.FLAG_FORCE_MFMA:
            flags |= _lib.FLAG_FORCE_GENERIC  # fp32 operands throughout (trittention_triton.py:92-98 of the reference)
        lib = _lib.lib()
        o = torch.empty_like(q)
        m = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
        with torch.cuda.device(q.device):
            ws = _lib.workspace(lib.tritt_dps_fwd_workspace_bytes(B, H, T, D, code, flags), q.device)
            st = lib.tritt_dps_fwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(m), B, H, T, D, code, float(softmax_scale), int(bool(causal)), k_diff,
                                   _lib.ptr(ws), ws.numel(), flags, _lib.stream_ptr(q.device))
        _lib.check(st, "tritt_dps_fwd")
        ctx.save_for_backward(q, k1, k2, v1, v2, o, m)
        ctx.causal = bool(causal)
        ctx.softmax_scale = float(softmax_scale)
        ctx.k_diff = k_diff
        ctx.flags = flags
        ctx.mark_non_differentiable(m)
        return o, m

    @staticmethod
    def backward(ctx, grad_output, m_grad=None):
        q, k1, k2, v1, v2, o, m = ctx.saved_tensors
        B, H, T, D = q.shape
        assert grad_output.shape == o.shape, f"Shape mismatch: O={o.shape}, dO={grad_output.shape}"
        assert o.device == grad_output.device, "O and dO must be on the same device"
        assert o.dtype == grad_output.dtype, "O and dO must have the same dtype"
        grad_output = _lib.dense(grad_output)
        lib = _lib.lib()
        code = _lib.dtype_code(q.dtype)
        dq, dk1, dk2, dv1, dv2 = (torch.empty_like(q) for _ in range(5))
        with torch.cuda.device(q.device):
            ws = _lib.workspace(lib.tritt_dps_bwd_workspace_bytes(B, H, T, D, code, ctx.flags), q.device)
            st = lib.tritt_dps_bwd(_lib.ptr(q), _lib.ptr(k1), _lib.ptr(k2), _lib.ptr(v1), _lib.ptr(v2), _lib.ptr(o),
                                   _lib.ptr(m), _lib.ptr(grad_output), _lib.ptr(dq), _lib.ptr(dk1), _lib.ptr(dk2),
                                   _lib.ptr(dv1), _lib.ptr(dv2), B, H, T, D, code, ctx.softmax_scale, int(ctx.causal),
                                   ctx.k_diff, _lib.ptr(ws), ws.numel(), ctx.flags, _lib.stream_ptr(q.device))
        _lib.check(st, "tritt_dps_bwd")
        return dq, dk1, dk2, dv1, dv2, None, None, None, None, None


class TrittentionTriton(nn.Module):
    def __init__(self, causal: bool = True, softmax_scale: float = 1 / 8, k_diff: int = 1024,
                 convert_to_float32: bool = False, input_precision: Optional[str] = None):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.k_diff = k_diff
        self.convert_to_float32 = convert_to_float32
        self.input_precision = input_precision

    _function = TrittentionTritonFunction

    def forward(self, q, k1, k2, v1, v2):
        """q, k1, k2, v1, v2: [B, N, S, D] -> (o [B, N, S, D], m [B, N, S] fp32 logsumexp)."""
        return self._function.apply(q, k1, k2, v1, v2, self.causal, self.softmax_scale, self.k_diff,
                                               self.convert_to_float32, self.input_precision)
