"""CPU oracle for the trittention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain dense PyTorch running on the CPU, the two
3-way attention formulations the library accelerates.  Only the test-suite,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it; the product path (the HIP library and its Python host code) never
does.

What each function follows in the reference:

* ``tdp_mask`` / ``tdp_forward_dense``:
  ``src/flash_trittention/triple_dot_product/trittention_pytorch.py:38-111``
  (mask :68-75, score einsum :81, flatten+scale :86-89, softmax :95,
  gated value :98-101) and ``kernels/utils.py:6-17`` (``None`` window = T).
* ``dps_mask`` / ``dps_forward_dense``:
  ``src/flash_trittention/dot_product_sum/trittention_pytorch.py:24-91``
  (mask :47-51 read by tensor axis, score :56-58, softmax :72, value :78-81).
* ``*_lse``: the log-sum-exp the fast path saves for backward
  (``triple_dot_product/flash_trittention.py:128``,
  ``dot_product_sum/kernels/fwd_kernel.py:366``): the true logsumexp of the
  scaled, masked scores (without the ``+0.01`` the naive modules add to their
  auxiliary ``L``; that term never reaches ``z``).
* gradients: ``torch.autograd`` of the dense forward, which is what the
  reference's tests compare against
  (``tests/test_triple_dot_product.py:83-96``).

Pinning (what the checks in ``tests/test_oracle.py`` hold each function to):
the reference ships no golden vectors for this path (its tests recompute both
sides at run time from CUDA RNG), so the oracle is pinned by mathematics:
T=1 closed form, Q=0 prefix-mean product, K2=1 reduction to
``scaled_dot_product_attention``, the float64 C brute force in
``oracle/brute_force.c`` (independent triple loops + analytic gradients),
finite differences, and for dot-product-sum the dense-vs-factorised identity
and the K1=0 reduction to biased SDPA.  The windowed-mask conventions
(``kk_left``/``kk_right``/``k1_window``/``k2_window``/``k_diff``) are pinned by
the committed fixture ``tests/golden/windowed_masks.npz``: outputs and all five
input gradients of the reference's own naive modules (float64, tiny shapes,
seven window settings for triple-dot and four ``k_diff`` values for
dot-product-sum), written by ``tests/golden/make_reference_vectors.py`` and
checked in ``tests/test_golden.py``.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

MASK_FILL = -1e6  # trittention_pytorch.py:110 (filled before the scale)


def _windows(T: int, k1_window, k2_window, kk_left, kk_right):
    """``None`` -> T (kernels/utils.py:13-16)."""
    f = lambda w: T if w is None else int(w)
    return f(k1_window), f(k2_window), f(kk_left), f(kk_right)


def tdp_mask(T: int, k1_window=None, k2_window=None, kk_left=None, kk_right=None,
             q_lo: int = 0, q_hi: Optional[int] = None, key_lo: int = 0,
             key_hi: Optional[int] = None) -> torch.Tensor:
    """Boolean [q, j, k] tensor, True = masked OUT (trittention_pytorch.py:68-75).

    Axis order here is (q, j, k) — the reference stores (j, k, q); the
    predicate is the same.  ``q_lo:q_hi`` selects a chunk of query rows,
    ``key_lo:key_hi`` the range of both key axes.
    """
    k1w, k2w, kl, kr = _windows(T, k1_window, k2_window, kk_left, kk_right)
    q_hi = T if q_hi is None else q_hi
    key_hi = T if key_hi is None else key_hi
    q = torch.arange(q_lo, q_hi).view(-1, 1, 1)
    j = torch.arange(key_lo, key_hi).view(1, -1, 1)
    k = torch.arange(key_lo, key_hi).view(1, 1, -1)
    return ((j > q) | (k > q) | (q > j + k1w) | (q > k + k2w)
            | (j + kl < k) | (k + kr < j))


def dps_mask(T: int, k_diff: int, q_lo: int = 0, q_hi: Optional[int] = None) -> torch.Tensor:
    """Boolean [q, s, t], True = masked OUT.

    dot_product_sum/trittention_pytorch.py:47-51, read by the axis each index
    tensor sits on: axis 2 of the [b,n,s,t,q] score is s (the K1 row), axis 3
    is t (the K2 row).  Valid iff s <= t <= q and t - s <= k_diff.
    """
    q_hi = T if q_hi is None else q_hi
    q = torch.arange(q_lo, q_hi).view(-1, 1, 1)
    s = torch.arange(T).view(1, -1, 1)
    t = torch.arange(T).view(1, 1, -1)
    return (s > t) | (t > q) | (t - s > k_diff)


def gated(v1, silu_dtype=None):
    """U = SiLU(V1).  The naive modules apply SiLU in the precision they compute in (fp32 in every comparison
    here).  The reference's kernel front-ends apply it in the TENSOR dtype before any kernel runs
    (triple_dot_product/flash_trittention.py:62, dot_product_sum/trittention_triton.py:55), so with 16-bit tensors
    their kernels see U rounded to 16 bit.  ``silu_dtype`` restates that rounding (straight-through for the
    gradient, which the front-ends also take as dU * SiLU'(V1), flash_trittention.py:389-391): the comparison
    target for tests that resolve differences below the 16-bit rounding of U itself."""
    u = F.silu(v1)
    if silu_dtype is not None:
        u = u + (u.detach().to(silu_dtype).to(u.dtype) - u.detach())
    return u


def _softmax_pv(score, masked, alpha, u, v2):
    """score [..., q, j, k] (unscaled) -> (z [..., q, d], lse [..., q])."""
    if masked is not None:
        score = score.masked_fill(masked, MASK_FILL)
    flat = score.flatten(-2) * alpha                      # [..., q, j*k]
    lse = torch.logsumexp(flat, dim=-1)
    p = torch.softmax(flat, dim=-1).view(score.shape)      # [..., q, j, k]
    t1 = torch.einsum("...qjk,...jd->...qkd", p, u)
    z = torch.einsum("...qkd,...kd->...qd", t1, v2)
    return z, lse


def tdp_forward_dense(q, k1, k2, v1, v2, alpha: float, causal: bool = True,
                      k1_window=None, k2_window=None, kk_left=None, kk_right=None, silu_dtype=None
                      ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Triple-dot-product forward, fully dense: returns (z, lse).

    q,k1,k2,v1,v2: [..., T, D] (any leading dims).  Differentiable.
    When ``causal`` is False no mask at all is applied and the windows are
    ignored (trittention_pytorch.py:83-84).
    """
    T = q.shape[-2]
    score = torch.einsum("...qd,...jd,...kd->...qjk", q, k1, k2)
    masked = tdp_mask(T, k1_window, k2_window, kk_left, kk_right) if causal else None
    return _softmax_pv(score, masked, alpha, gated(v1, silu_dtype), v2)


def dps_forward_dense(q, k1, k2, v1, v2, alpha: float, causal: bool = True,
                      k_diff: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dot-product-sum forward, fully dense over the [q, s, t] cube: (z, lse)."""
    T = q.shape[-2]
    k_diff = T if k_diff is None else int(k_diff)
    qk = torch.einsum("...qd,...td->...qt", q, k2)          # [.., q, t]
    kk = torch.einsum("...sd,...td->...st", k1, k2)          # [.., s, t]
    score = qk.unsqueeze(-2) + kk.unsqueeze(-3)              # [.., q, s, t]
    masked = dps_mask(T, k_diff) if causal else None
    return _softmax_pv(score, masked, alpha, F.silu(v1), v2)


def dps_forward_factorised(q, k1, k2, v1, v2, alpha: float, causal: bool = True,
                           k_diff: Optional[int] = None):
    """Dot-product-sum as two chained softmaxes (O(T^2 D)); returns (z, lse).

    exp(alpha (Q_q.K2_t + K1_s.K2_t)) factorises and the mask never couples s
    with q, so  lse1[t] = logsumexp_s alpha K1_s.K2_t,  R[t] = softmax_s @ U,
    then an ordinary attention of Q over K2 with per-key bias lse1[t] and
    values R[t]*V2[t].  (The reference's fast kernel uses the same structure:
    dot_product_sum/kernels/fwd_kernel.py:102-218.)  Cross-checked against
    ``dps_forward_dense`` in the tests; used where the dense cube is too big.
    """
    T = q.shape[-2]
    k_diff = T if k_diff is None else int(k_diff)
    a = torch.einsum("...td,...sd->...ts", k2, k1) * alpha   # [.., t, s]
    if causal:
        t = torch.arange(T).view(-1, 1)
        s = torch.arange(T).view(1, -1)
        a = a.masked_fill((s > t) | (t - s > k_diff), float("-inf"))
    lse1 = torch.logsumexp(a, dim=-1)                        # [.., t]
    r = torch.softmax(a, dim=-1) @ F.silu(v1)                # [.., t, d]
    b = torch.einsum("...qd,...td->...qt", q, k2) * alpha + lse1.unsqueeze(-2)
    if causal:
        qi = torch.arange(T).view(-1, 1)
        ti = torch.arange(T).view(1, -1)
        b = b.masked_fill(ti > qi, float("-inf"))
    lse = torch.logsumexp(b, dim=-1)
    z = torch.softmax(b, dim=-1) @ (r * v2)
    return z, lse


def _grads(fn, inputs, d_out):
    leaves = [t.detach().clone().requires_grad_(True) for t in inputs]
    z, lse = fn(*leaves)
    z.backward(d_out)
    return z.detach(), lse.detach(), [t.grad for t in leaves]


def tdp_forward_backward(q, k1, k2, v1, v2, d_out, alpha, causal=True, **windows):
    """(z, lse, [dq, dk1, dk2, dv1, dv2]) via autograd of the dense forward."""
    fn = lambda *a: tdp_forward_dense(*a, alpha=alpha, causal=causal, **windows)
    return _grads(fn, (q, k1, k2, v1, v2), d_out)


def dps_forward_backward(q, k1, k2, v1, v2, d_out, alpha, causal=True, k_diff=None,
                         factorised=False):
    f = dps_forward_factorised if factorised else dps_forward_dense
    fn = lambda *a: f(*a, alpha=alpha, causal=causal, k_diff=k_diff)
    return _grads(fn, (q, k1, k2, v1, v2), d_out)


def tdp_forward_backward_chunked(q, k1, k2, v1, v2, d_out, alpha, causal=True,
                                 q_chunk: int = 64, need_grads: bool = True, rows=None, **windows):
    """Same as ``tdp_forward_backward`` for ONE head ([T, D] inputs),
    evaluated in chunks of query rows so the [q, j, k] slab stays small
    (T=1024: 64 x 1024 x 1024 fp32 = 268 MB).  For a causal chunk only
    j,k <= last query of the chunk are touched, and under windows only keys
    from (first query of the chunk - the larger query window) on: the keys
    left out are masked for every query of the chunk, and a masked score
    contributes an exact zero to the dense softmax.  ``rows=(lo, hi)``
    (forward only) evaluates just the query rows lo..hi-1 and returns
    [hi - lo, ...] tensors: spot checks at sequence lengths whose full plane
    is out of reach.
    """
    assert q.dim() == 2
    T, D = q.shape
    r_lo, r_hi = rows if rows is not None else (0, T)
    assert rows is None or not need_grads
    leaves = [t.detach().clone().requires_grad_(need_grads) for t in (q, k1, k2, v1, v2)]
    ql, k1l, k2l, v1l, v2l = leaves
    z_out = torch.empty_like(q[r_lo:r_hi])
    lse_out = torch.empty(r_hi - r_lo, dtype=q.dtype)
    k1w, k2w, _, _ = _windows(T, windows.get("k1_window"), windows.get("k2_window"), None, None)
    for lo in range(r_lo, r_hi, q_chunk):
        hi = min(r_hi, lo + q_chunk)
        n = hi if causal else T          # keys beyond the chunk's last query are masked
        ks = max(0, lo - max(k1w, k2w)) if causal else 0
        with torch.set_grad_enabled(need_grads):
            u = F.silu(v1l[ks:n])
            qk1 = ql[lo:hi, None, :] * k1l[None, ks:n, :]            # [c, n - ks, D]
            score = qk1 @ k2l[ks:n].t()                              # [c, j, k]
            if causal:
                masked = tdp_mask(T, q_lo=lo, q_hi=hi, key_lo=ks, key_hi=n, **windows)
                score = score.masked_fill(masked, MASK_FILL)
            flat = score.flatten(-2) * alpha
            lse = torch.logsumexp(flat, dim=-1)
            p = torch.softmax(flat, dim=-1).view(score.shape)
            t1 = torch.einsum("qjk,jd->qkd", p, u)
            z = (t1 * v2l[None, ks:n, :]).sum(1)
            if need_grads:
                z.backward(d_out[lo:hi])
        z_out[lo - r_lo:hi - r_lo] = z.detach()
        lse_out[lo - r_lo:hi - r_lo] = lse.detach()
    grads = [t.grad for t in leaves] if need_grads else None
    return z_out, lse_out, grads


def make_inputs(B, H, T, D, dtype=torch.float32, seed=0, n=6):
    """Seeded inputs shared by the tests, smoke() and bench: six N(0,1) draws
    from a CPU generator in the order Q, K1, K2, V1, V2, dO, drawn in fp32 and
    then cast to ``dtype`` (so the oracle and the device path see the same
    already-rounded values)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    return [torch.randn(B, H, T, D, generator=g, dtype=torch.float32).to(dtype)
            for _ in range(n)]


def default_alpha(D: int) -> float:
    return 1.0 / math.sqrt(D)
