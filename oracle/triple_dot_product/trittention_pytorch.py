"""``Trittention_pytorch`` for the triple-dot-product variant.  TEST INFRASTRUCTURE ONLY.

A dense CPU ``nn.Module`` with the constructor, call signature and return tuple of the reference's
naive module (``src/flash_trittention/triple_dot_product/trittention_pytorch.py:10-102``), so the
reference's own tests and scripts (``tests/test_triple_dot_product.py:13-17``) can be pointed at
it.  It is built on the oracle's functions (``oracle/trittention_oracle.py``); the product package
never imports it.

Returns ``(z, pre_softmax, v_gated, M, L)`` (reference :102):
* ``z [B,H,T,D]``: the attention output;
* ``pre_softmax [B,H,j,k,q]``: the unscaled scores with masked entries set to -1e6 (:81, :110),
  key axes first and the query axis last as the reference stores them;
* ``v_gated [B,H,j,k,D] = SiLU(V1[j]) * V2[k]`` (:98-99);
* ``M [B,H,T]``: the row maximum of the scaled scores (:92);
* ``L [B,H,T] = sum exp(scaled score - M) + 0.01`` (:94; the 0.01 is the reference's).

Pinned by ``tests/golden/windowed_masks.npz`` (all five returns of the reference module on seven
window settings; ``tests/test_golden.py``).
"""
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import trittention_oracle as orc


class Trittention_pytorch(nn.Module):
    def __init__(self, causal: bool = True, softmax_scale: float = 1 / 8, n_ctx: int = 1024,
                 k1_window: Optional[int] = None, k2_window: Optional[int] = None,
                 kk_left: Optional[int] = None, kk_right: Optional[int] = None):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.n_ctx = n_ctx
        # None = n_ctx (kernels/utils.py:13-16); the mask itself is rebuilt per call for the actual T
        self.k1_window, self.k2_window, self.kk_left, self.kk_right = orc._windows(
            n_ctx, k1_window, k2_window, kk_left, kk_right)

    def forward(self, q, k1, k2, v1, v2):
        T = q.shape[-2]
        if T > self.n_ctx:
            raise ValueError(f"sequence length {T} exceeds n_ctx={self.n_ctx}")
        score = torch.einsum("bhqd,bhjd,bhkd->bhqjk", q, k1, k2)
        if self.causal:
            masked = orc.tdp_mask(T, self.k1_window, self.k2_window, self.kk_left, self.kk_right)
            score = score.masked_fill(masked.to(score.device), orc.MASK_FILL)
        flat = score.flatten(-2) * self.softmax_scale
        M = flat.amax(dim=-1)
        L = torch.exp(flat - M.unsqueeze(-1)).sum(dim=-1) + 0.01
        p = torch.softmax(flat, dim=-1).view(score.shape)
        v_gated = F.silu(v1).unsqueeze(3) * v2.unsqueeze(2)          # [b,h,j,k,d]
        z = torch.einsum("bhqjk,bhjkd->bhqd", p, v_gated)
        return z, score.permute(0, 1, 3, 4, 2), v_gated, M, L
