"""Triple-dot-product trittention on MI355X.

Mirrors the reference's ``FlashTrittention`` autograd Function and the public
``flash_trittention`` (triple_dot_product/flash_trittention.py:14-139 forward,
:141-393 backward, :396-438 entry point): same argument order, defaults,
return values and ValueErrors.  The work itself is one call into the HIP
library per direction (SiLU, Delta and SiLU' are done inside it).
"""
import warnings
from typing import Optional

import torch
import torch.nn as nn

from .. import _lib, _ops
from .utils import process_masking_variables


def _validate(Q, others):
    for name, t in others:
        if t.shape != Q.shape:
            raise ValueError(f"{name} shape {tuple(t.shape)} does not match Q shape {tuple(Q.shape)}")
        if t.dtype != Q.dtype:
            raise ValueError(f"{name} dtype {t.dtype} does not match Q dtype {Q.dtype}")
        if t.device != Q.device:
            raise ValueError(f"{name} device {t.device} does not match Q device {Q.device}")
    if Q.dim() != 4:
        raise ValueError(f"expected [batch, heads, seq_len, head_dim] tensors, got shape {tuple(Q.shape)}")
    head_dim = Q.shape[-1]
    if head_dim <= 0 or head_dim & (head_dim - 1):
        raise ValueError(f"head_dim must be a power of 2, got {head_dim}")
    if head_dim not in (8, 16, 32, 64, 128):
        raise ValueError(f"head_dim must be one of 8, 16, 32, 64, 128, got {head_dim}")
    _lib.dtype_code(Q.dtype)


class FlashTrittention(torch.autograd.Function):
    # `flags` of the C ABI (_lib.FLAG_*).  A constant of the class, never assigned to: a caller that wants
    # another implementation uses the subclass `with_flags(flags)` returns.
    IMPL_FLAGS = _lib.FLAG_AUTO

    @classmethod
    def with_flags(cls, flags: int):
        """The Function whose calls pass `flags` to the library (tests pin the fp32 or the MFMA kernels)."""
        return _lib.flagged_subclass(cls, flags)

    @staticmethod
    def forward(ctx, Q, K1, K2, V1, V2, softmax_scale, kk_left, kk_right, k1_window, k2_window, causal,
                convert_to_float32):
        _validate(Q, (("K1", K1), ("K2", K2), ("V1", V1), ("V2", V2)))
        T = Q.shape[2]
        k1_window, k2_window, kk_left, kk_right = process_masking_variables(T, k1_window, k2_window, kk_left, kk_right)
        causal = bool(causal)
        compiling = _ops.compiling()  # tracing: the implementation flags are the class default
        # views the library can read where they lie ([B,T,H,D] transposed, slices of a fused projection) stay as they
        # are, and are what the backward gets; the rest is copied, as the reference copies every input
        # (flash_trittention.py:64-68)
        Q, K1, K2, V1, V2 = (t.contiguous() if compiling else _lib.view(t) for t in (Q, K1, K2, V1, V2))
        flags = _lib.FLAG_AUTO if compiling else getattr(getattr(ctx, "_forward_cls", None), "IMPL_FLAGS", _lib.FLAG_AUTO)
        if torch.are_deterministic_algorithms_enabled():
            flags &= ~_lib.FLAG_FLOAT_ATOMICS  # the default (fixed-point accumulation) is bitwise reproducible
        if convert_to_float32 and not flags & (_lib.FLAG_FORCE_MFMA | _lib.FLAG_FORCE_GENERIC):
            # the reference upcasts the operands of its score products under this flag (flash_trittention.py:408,
            # bwd_dq.py:197,219).  16-bit tensors with D = 32 or 64 stay on the matrix cores with those operands
            # kept to 16 mantissa bits (hi + lo pairs); other shapes take the fp32 kernels
            if Q.dtype != torch.float32 and Q.shape[-1] in (32, 64):
                flags |= _lib.FLAG_SPLIT_OPERANDS
            else:
                flags |= _lib.FLAG_FORCE_GENERIC
        call = torch.ops.flash_trittention.tdp_fwd if compiling else _ops.tdp_fwd_impl
        O, LSE = call(Q, K1, K2, V1, V2, float(softmax_scale), causal, k1_window, k2_window, kk_left, kk_right, flags)
        ctx.save_for_backward(Q, K1, K2, V1, V2, O, LSE)  # split operands: O is [2,B,H,T,D], output and residual
        if flags & _lib.FLAG_SPLIT_OPERANDS:
            O = O[0]
        ctx.softmax_scale = float(softmax_scale)
        ctx.windows = (k1_window, k2_window, kk_left, kk_right)
        ctx.causal = causal
        ctx.flags = flags
        return O

    @staticmethod
    def backward(ctx, dO):
        Q, K1, K2, V1, V2, O, LSE = ctx.saved_tensors
        if dO.dtype != Q.dtype:
            dO = dO.to(Q.dtype)
        if _ops.compiling():
            dO = dO.contiguous()
        k1_window, k2_window, kk_left, kk_right = ctx.windows
        # only the gradients autograd asks for: the library skips the others (and the kernel launch that serves
        # nothing else)
        needs = getattr(ctx, "needs_input_grad", (True,) * 5)
        wanted = sum(1 << i for i in range(5) if needs[i])
        if _ops.compiling():
            grads = torch.ops.flash_trittention.tdp_bwd(Q, K1, K2, V1, V2, O, LSE, dO, ctx.softmax_scale, ctx.causal,
                                                        k1_window, k2_window, kk_left, kk_right, ctx.flags, wanted)
            grads = [g if needs[i] else None for i, g in enumerate(grads)]
        else:
            grads = _ops.tdp_bwd_impl(Q, K1, K2, V1, V2, O, LSE, dO, ctx.softmax_scale, ctx.causal, k1_window, k2_window,
                                      kk_left, kk_right, ctx.flags, wanted)
        return (*grads, None, None, None, None, None, None, None)


def flash_trittention(q, k1, k2, v1, v2, softmax_scale=1 / 8, kk_left=1, kk_right=1, k1_window=1, k2_window=1,
                      causal=True, convert_to_float32=False, input_precision=None):
    """Triple-dot-product 3-way attention; returns O [B, H, T, D].

    Window arguments: ``None`` (or any value >= seq_len) disables a window; note that the
    literal defaults are 1, a narrow band, exactly as in the reference.  Softmax and accumulation are
    always fp32.  ``convert_to_float32=True`` also keeps the operands of the score products beyond 16-bit
    rounding: for 16-bit tensors with head_dim 32 or 64 as hi + lo pairs on the matrix cores (about 1.4 times
    the default path's time), otherwise on the fp32 kernels.  Scores spanning hundreds then keep the full
    16-bit tolerance, where the 16-bit operands of the default path do not.
    ``input_precision`` is accepted and ignored with a warning, as in the reference.
    """
    if input_precision is not None:
        warnings.warn(
            "flash_trittention: `input_precision` is currently unused and has no effect "
            f"(got {input_precision!r}).", stacklevel=2)
    return FlashTrittention.apply(q, k1, k2, v1, v2, softmax_scale, kk_left, kk_right, k1_window, k2_window, causal,
                                  convert_to_float32)


class FlashTrittentionModule(nn.Module):
    """``nn.Module`` front of ``flash_trittention`` (the triple-dot counterpart of ``TrittentionTriton``).

    The constructor takes what the reference's naive module takes
    (triple_dot_product/trittention_pytorch.py:12-21: causal, softmax_scale, n_ctx and the four windows, ``None`` =
    no window), so a model built on ``Trittention_pytorch`` can swap the class; ``n_ctx`` is accepted and only
    checked (no mask is precomputed).  ``forward`` returns O [B, H, T, D] alone: the dense score and gated-value
    tensors the naive module also returns are never formed here."""

    def __init__(self, causal: bool = True, softmax_scale: float = 1 / 8, n_ctx: Optional[int] = None,
                 k1_window: Optional[int] = None, k2_window: Optional[int] = None, kk_left: Optional[int] = None,
                 kk_right: Optional[int] = None, convert_to_float32: bool = False):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.n_ctx = n_ctx
        self.k1_window, self.k2_window, self.kk_left, self.kk_right = k1_window, k2_window, kk_left, kk_right
        self.convert_to_float32 = convert_to_float32

    def forward(self, q, k1, k2, v1, v2):
        if self.n_ctx is not None and q.shape[-2] > self.n_ctx:
            raise ValueError(f"sequence length {q.shape[-2]} exceeds n_ctx={self.n_ctx}")
        return flash_trittention(q, k1, k2, v1, v2, softmax_scale=self.softmax_scale, kk_left=self.kk_left,
                                 kk_right=self.kk_right, k1_window=self.k1_window, k2_window=self.k2_window,
                                 causal=self.causal, convert_to_float32=self.convert_to_float32)

    def extra_repr(self):
        return (f"causal={self.causal}, softmax_scale={self.softmax_scale}, windows="
                f"({self.k1_window}, {self.k2_window}, {self.kk_left}, {self.kk_right})")
