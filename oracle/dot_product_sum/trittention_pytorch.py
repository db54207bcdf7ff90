"""``Trittention_pytorch`` for the dot-product-sum variant.  TEST INFRASTRUCTURE ONLY.

A dense CPU ``nn.Module`` with the constructor, call signature and return tuple of the reference's
naive module (``src/flash_trittention/dot_product_sum/trittention_pytorch.py:8-82``), built on the
oracle's functions; the product package never imports it.

Returns ``(z, pre_softmax, v_gated, M)`` (reference :82):
* ``z [B,H,T,D]``;
* ``pre_softmax [B,H,s,t,q]``: the unscaled scores ``K2[t].Q[q] + K1[s].K2[t]`` with masked entries
  set to -1e6 (:56-58, :90);
* ``v_gated [B,H,s,t,D] = SiLU(V1[s]) * V2[t]`` (:78-79);
* ``M [B,H,T] = rowmax + log(sum exp(scaled score - rowmax) + 0.01)`` (:69-74; a log-sum-exp that
  carries the reference's 0.01).

Pinned by ``tests/golden/windowed_masks.npz`` (all four returns of the reference module on four
``k_diff`` settings; ``tests/test_golden.py``).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import trittention_oracle as orc


class Trittention_pytorch(nn.Module):
    def __init__(self, causal: bool = True, softmax_scale: float = 1 / 8, n_ctx: int = 1024, k_diff: int = 1024):
        super().__init__()
        self.causal = causal
        self.softmax_scale = softmax_scale
        self.n_ctx = n_ctx
        self.k_diff = k_diff

    def forward(self, q, k1, k2, v1, v2):
        T = q.shape[-2]
        if T > self.n_ctx:
            raise ValueError(f"sequence length {T} exceeds n_ctx={self.n_ctx}")
        qk = torch.einsum("bhqd,bhtd->bhqt", q, k2)
        kk = torch.einsum("bhsd,bhtd->bhst", k1, k2)
        score = qk.unsqueeze(-2) + kk.unsqueeze(-3)                  # [b,h,q,s,t]
        if self.causal:
            score = score.masked_fill(orc.dps_mask(T, self.k_diff).to(score.device), orc.MASK_FILL)
        flat = score.flatten(-2) * self.softmax_scale
        rowmax = flat.amax(dim=-1)
        M = rowmax + torch.log(torch.exp(flat - rowmax.unsqueeze(-1)).sum(dim=-1) + 0.01)
        p = torch.softmax(flat, dim=-1).view(score.shape)
        v_gated = F.silu(v1).unsqueeze(3) * v2.unsqueeze(2)          # [b,h,s,t,d]
        z = torch.einsum("bhqst,bhstd->bhqd", p, v_gated)
        return z, score.permute(0, 1, 3, 4, 2), v_gated, M
