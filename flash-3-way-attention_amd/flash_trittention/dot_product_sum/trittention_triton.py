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

from .. import _lib, _ops
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
        if D not in (8, 16, 32, 64, 128):
            raise ValueError(f"head_dim must be one of 8, 16, 32, 64, 128, got {D}")
        _lib.dtype_code(q.dtype)
        k_diff = clamp_window(k_diff, T, "k_diff")
        compiling = _ops.compiling()
        # views the library can read where they lie stay as they are (and are what the backward gets); the rest is
        # copied, as the reference copies every input (trittention_triton.py:43-47)
        q, k1, k2, v1, v2 = (t.contiguous() if compiling else _lib.view(t) for t in (q, k1, k2, v1, v2))
        flags = _lib.FLAG_AUTO if compiling else getattr(getattr(ctx, "_forward_cls", None), "IMPL_FLAGS", _lib.FLAG_AUTO)
        if convert_to_float32 and not flags & _lib.FLAG_FORCE_MFMA:
            flags |= _lib.FLAG_FORCE_GENERIC  # fp32 operands throughout (trittention_triton.py:92-98 of the reference)
        call = torch.ops.flash_trittention.dps_fwd if compiling else _ops.dps_fwd_impl
        o, m = call(q, k1, k2, v1, v2, float(softmax_scale), bool(causal), k_diff, flags)
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
        assert grad_output.shape == o.shape, f"Shape mismatch: O={o.shape}, dO={grad_output.shape}"
        assert o.device == grad_output.device, "O and dO must be on the same device"
        assert o.dtype == grad_output.dtype, "O and dO must have the same dtype"
        if _ops.compiling():
            grad_output = grad_output.contiguous()
        call = torch.ops.flash_trittention.dps_bwd if _ops.compiling() else _ops.dps_bwd_impl
        dq, dk1, dk2, dv1, dv2 = call(q, k1, k2, v1, v2, o, m, grad_output, ctx.softmax_scale, ctx.causal, ctx.k_diff,
                                      ctx.flags)
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
