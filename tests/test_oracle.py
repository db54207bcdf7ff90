"""Pins the CPU oracle (oracle/) with mathematics, since the reference ships
no golden vectors for this path: closed forms, a library routine
(scaled_dot_product_attention), an independent float64 C brute force with
analytic gradients, and finite differences.  Each check is chosen so that a
plausible slip (dropped scale, swapped j/k, wrong mask side, missing SiLU,
wrong sign in dS) fails at least one of them."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute
from oracle import trittention_oracle as orc

torch.manual_seed(0)
DT = torch.float64


def rnd(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=DT)


def prefix_mean(x):
    T = x.shape[-2]
    return x.cumsum(-2) / torch.arange(1, T + 1, dtype=x.dtype).view(-1, 1)


# ------------------------------------------------------------------ closed forms
def test_tdp_T1_is_gated_value():
    q, k1, k2, v1, v2 = (rnd(2, 1, 8, seed=s) for s in range(5))
    z, lse = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=0.3)
    assert torch.allclose(z, F.silu(v1) * v2, atol=1e-14)
    assert torch.allclose(lse, 0.3 * (q * k1 * k2).sum(-1), atol=1e-14)


def test_tdp_zero_query_gives_product_of_prefix_means():
    T, D = 11, 5
    q = torch.zeros(T, D, dtype=DT)
    k1, k2, v1, v2 = (rnd(T, D, seed=s) for s in range(1, 5))
    z, lse = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=0.7)
    assert torch.allclose(z, prefix_mean(F.silu(v1)) * prefix_mean(v2), atol=1e-13)
    n = torch.arange(1, T + 1, dtype=DT)
    assert torch.allclose(lse, 2 * torch.log(n), atol=1e-13)


@pytest.mark.parametrize("which", ["k2", "k1"])
def test_tdp_ones_key_reduces_to_sdpa(which):
    """K2 = 1 => s = alpha Q.K1_j: ordinary causal attention over (K1, U) times
    the prefix mean of V2 (and symmetrically for K1 = 1)."""
    T, D = 13, 8
    q, k1, k2, v1, v2 = (rnd(T, D, seed=10 + s) for s in range(5))
    alpha = 0.41
    if which == "k2":
        k2 = torch.ones_like(k2)
        sd = F.scaled_dot_product_attention(q[None], k1[None], F.silu(v1)[None],
                                            is_causal=True, scale=alpha)[0]
        want = sd * prefix_mean(v2)
    else:
        k1 = torch.ones_like(k1)
        sd = F.scaled_dot_product_attention(q[None], k2[None], v2[None],
                                            is_causal=True, scale=alpha)[0]
        want = sd * prefix_mean(F.silu(v1))
    z, _ = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=alpha)
    assert torch.allclose(z, want, atol=1e-12)


def test_tdp_constant_values_and_shift_invariance():
    T, D = 9, 4
    q, k1, k2 = (rnd(T, D, seed=s) for s in range(3))
    c = 1.2784645  # silu(c) computed below
    v1 = torch.full((T, D), c, dtype=DT)
    v2 = torch.ones(T, D, dtype=DT)
    z, _ = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=1.0)
    assert torch.allclose(z, F.silu(v1), atol=1e-13)


def test_noncausal_ignores_windows_and_mask():
    T, D = 7, 4
    q, k1, k2, v1, v2 = (rnd(T, D, seed=20 + s) for s in range(5))
    z0, _ = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=0.5, causal=False)
    z1, _ = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=0.5, causal=False,
                                  k1_window=1, k2_window=1, kk_left=0, kk_right=0)
    assert torch.equal(z0, z1)
    s = torch.einsum("qd,jd,kd->qjk", q, k1, k2).flatten(1) * 0.5
    v = (F.silu(v1)[:, None, :] * v2[None, :, :]).flatten(0, 1)
    assert torch.allclose(z0, torch.softmax(s, -1) @ v, atol=1e-13)


# ------------------------------------------------------------------ C brute force
WINDOW_CASES = [(None, None, None, None), (5, 3, 4, 1), (2, 7, 0, 3), (100, 100, 1, 1)]


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("win", WINDOW_CASES)
def test_tdp_oracle_matches_float64_brute_force(causal, win):
    T, D, alpha = 12, 4, 0.37
    q, k1, k2, v1, v2, do = (rnd(T, D, seed=30 + s) for s in range(6))
    kw = dict(zip(("k1_window", "k2_window", "kk_left", "kk_right"), win))
    z, lse, grads = orc.tdp_forward_backward(q, k1, k2, v1, v2, do, alpha, causal, **kw)
    w = [T if x is None else x for x in win]
    ref = brute.brute(0, *(t.numpy() for t in (q, k1, k2, v1, v2, do)), alpha, causal, w)
    assert np.allclose(z.numpy(), ref[0], atol=1e-12)
    assert np.allclose(lse.numpy(), ref[1], atol=1e-12)
    for g, r, name in zip(grads, ref[2:], ("dq", "dk1", "dk2", "dv1", "dv2")):
        assert np.allclose(g.numpy(), r, atol=1e-11), name


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("k_diff", [None, 2, 5, 0])
@pytest.mark.parametrize("factorised", [False, True])
def test_dps_oracle_matches_float64_brute_force(causal, k_diff, factorised):
    T, D, alpha = 12, 4, 0.37
    q, k1, k2, v1, v2, do = (rnd(T, D, seed=40 + s) for s in range(6))
    z, lse, grads = orc.dps_forward_backward(q, k1, k2, v1, v2, do, alpha, causal,
                                             k_diff=k_diff, factorised=factorised)
    ref = brute.brute(1, *(t.numpy() for t in (q, k1, k2, v1, v2, do)), alpha, causal,
                      [T if k_diff is None else k_diff])
    assert np.allclose(z.numpy(), ref[0], atol=1e-12)
    assert np.allclose(lse.numpy(), ref[1], atol=1e-12)
    for g, r, name in zip(grads, ref[2:], ("dq", "dk1", "dk2", "dv1", "dv2")):
        assert np.allclose(g.numpy(), r, atol=1e-11), name


def test_brute_force_gradients_match_finite_differences():
    """The C analytic gradients themselves are pinned by central differences
    of the C forward (so brute force and autograd are not merely agreeing on
    a shared misreading of the formulas)."""
    T, D, alpha = 5, 3, 0.6
    arrs = [rnd(T, D, seed=50 + s).numpy() for s in range(6)]
    for variant, w in ((0, [T, T, T, T]), (0, [3, 2, 1, 2]), (1, [T]), (1, [1])):
        out = brute.brute(variant, *arrs, alpha, True, w)
        for idx, g in enumerate(out[2:]):
            num = np.zeros_like(g)
            for i in range(T):
                for d in range(D):
                    eps = 1e-6
                    ap = [a.copy() for a in arrs]
                    am = [a.copy() for a in arrs]
                    ap[idx][i, d] += eps
                    am[idx][i, d] -= eps
                    zp = brute.brute(variant, *ap, alpha, True, w)[0]
                    zm = brute.brute(variant, *am, alpha, True, w)[0]
                    num[i, d] = ((zp - zm) * arrs[5]).sum() / (2 * eps)
            assert np.allclose(g, num, atol=1e-7), (variant, w, idx)


# ------------------------------------------------------------------ dps closed forms
def test_dps_zero_k1_reduces_to_biased_sdpa():
    """K1 = 0: inner softmax is uniform over s<=t, so the outer pass is plain
    attention of Q over K2 with bias log(t+1) and values prefixmean(U)*V2."""
    T, D, alpha = 10, 6, 0.45
    q, _, k2, v1, v2 = (rnd(T, D, seed=60 + s) for s in range(5))
    k1 = torch.zeros(T, D, dtype=DT)
    z, lse = orc.dps_forward_dense(q, k1, k2, v1, v2, alpha=alpha)
    bias = torch.log(torch.arange(1, T + 1, dtype=DT)).view(1, -1).expand(T, T)
    causal = torch.full((T, T), float("-inf"), dtype=DT).triu(1)
    want = F.scaled_dot_product_attention(q[None], k2[None], (prefix_mean(F.silu(v1)) * v2)[None],
                                          attn_mask=(bias + causal)[None], scale=alpha)[0]
    assert torch.allclose(z, want, atol=1e-12)


def test_dps_T1():
    q, k1, k2, v1, v2 = (rnd(1, 8, seed=70 + s) for s in range(5))
    z, lse = orc.dps_forward_dense(q, k1, k2, v1, v2, alpha=0.3)
    assert torch.allclose(z, F.silu(v1) * v2, atol=1e-14)
    assert torch.allclose(lse, 0.3 * (k2 * (q + k1)).sum(-1), atol=1e-14)


# ------------------------------------------------------------------ chunked == dense
@pytest.mark.parametrize("causal", [True, False])
def test_chunked_equals_dense(causal):
    T, D, alpha = 40, 8, 0.35
    q, k1, k2, v1, v2, do = (rnd(T, D, seed=80 + s) for s in range(6))
    z, lse, g = orc.tdp_forward_backward(q, k1, k2, v1, v2, do, alpha, causal)
    zc, lsec, gc = orc.tdp_forward_backward_chunked(q, k1, k2, v1, v2, do, alpha, causal, q_chunk=16)
    assert torch.allclose(z, zc, atol=1e-12) and torch.allclose(lse, lsec, atol=1e-12)
    for a, b in zip(g, gc):
        assert torch.allclose(a, b, atol=1e-11)


@pytest.mark.parametrize("causal", [True, False])
def test_chunked_row_range_equals_dense_rows(causal):
    T, D, alpha = 40, 8, 0.35
    q, k1, k2, v1, v2 = (rnd(T, D, seed=85 + s) for s in range(5))
    z, lse = orc.tdp_forward_dense(q, k1, k2, v1, v2, alpha=alpha, causal=causal)
    zr, lser, g = orc.tdp_forward_backward_chunked(q, k1, k2, v1, v2, None, alpha, causal, q_chunk=7,
                                                   need_grads=False, rows=(11, 30))
    assert g is None and zr.shape == (19, D)
    assert torch.allclose(z[11:30], zr, atol=1e-12) and torch.allclose(lse[11:30], lser, atol=1e-12)


@pytest.mark.parametrize("windows", [(5, 3, 4, 1), (2, 30, 0, 3), (12, 12, 40, 40)])
def test_chunked_with_windows_equals_dense(windows):
    T, D, alpha = 40, 8, 0.35
    kw = dict(zip(("k1_window", "k2_window", "kk_left", "kk_right"), windows))
    q, k1, k2, v1, v2, do = (rnd(T, D, seed=70 + s) for s in range(6))
    z, lse, g = orc.tdp_forward_backward(q, k1, k2, v1, v2, do, alpha, True, **kw)
    zc, lsec, gc = orc.tdp_forward_backward_chunked(q, k1, k2, v1, v2, do, alpha, True, q_chunk=7, **kw)
    assert torch.allclose(z, zc, atol=1e-12) and torch.allclose(lse, lsec, atol=1e-12)
    for a, b in zip(g, gc):
        assert torch.allclose(a, b, atol=1e-11)


def test_batched_heads_are_independent():
    B, H, T, D = 2, 3, 9, 4
    ins = [rnd(B, H, T, D, seed=90 + s) for s in range(5)]
    z, lse = orc.tdp_forward_dense(*ins, alpha=0.5)
    z11, lse11 = orc.tdp_forward_dense(*(t[1, 2] for t in ins), alpha=0.5)
    assert torch.allclose(z[1, 2], z11, atol=1e-13) and torch.allclose(lse[1, 2], lse11, atol=1e-13)


def test_make_inputs_is_seeded_and_ordered():
    a = orc.make_inputs(1, 2, 4, 8, seed=3)
    b = orc.make_inputs(1, 2, 4, 8, seed=3)
    assert len(a) == 6 and all(torch.equal(x, y) for x, y in zip(a, b))
    g = torch.Generator().manual_seed(3)
    assert torch.equal(a[0], torch.randn(1, 2, 4, 8, generator=g))


def test_rounded_silu_is_the_dense_formula_on_rounded_gated_values():
    """`silu_dtype` only replaces U = SiLU(V1) by its rounding (the forward equals the softmax-weighted sum with
    that U passed in directly) and leaves the gradient path through SiLU'(V1) in place (straight-through: dV1 =
    dU * SiLU'(V1) with dU taken at the rounded U)."""
    q, k1, k2, v1, v2, do = (t[0, 0] for t in orc.make_inputs(1, 1, 20, 8, torch.float32, seed=3))
    z, lse = orc.tdp_forward_dense(q, k1, k2, v1, v2, 0.3, True, silu_dtype=torch.bfloat16)
    u = torch.nn.functional.silu(v1).bfloat16().float()
    assert not torch.equal(u, torch.nn.functional.silu(v1))
    score = torch.einsum("qd,jd,kd->qjk", q, k1, k2)
    z2, lse2 = orc._softmax_pv(score, orc.tdp_mask(20), 0.3, u, v2)
    assert torch.equal(z, z2) and torch.equal(lse, lse2)
    # gradient: dV1 = dU * SiLU'(V1), dU from the formula evaluated at the rounded U
    _, _, g = orc.tdp_forward_backward(q, k1, k2, v1, v2, do, 0.3, True, silu_dtype=torch.bfloat16)
    ul = u.clone().requires_grad_(True)
    z3, _ = orc._softmax_pv(score, orc.tdp_mask(20), 0.3, ul, v2)
    z3.backward(do)
    sg = torch.sigmoid(v1)
    torch.testing.assert_close(g[3], ul.grad * sg * (1 + v1 * (1 - sg)), rtol=1e-6, atol=1e-7)
