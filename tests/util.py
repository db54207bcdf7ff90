"""Shared helpers for the GPU parity tests: seeded CPU inputs, oracle results,
and runners that go through the Python host -> ctypes -> C ABI -> HIP path."""
import torch

from oracle import trittention_oracle as orc

NAMES = ("dq", "dk1", "dk2", "dv1", "dv2")


def oracle_tdp(inputs, alpha, causal, windows=(None,) * 4, per_head=True, silu_dtype=None):
    """Oracle in fp32 on the already-rounded inputs (what the reference's tests do:
    tests/test_triple_dot_product.py:47).  Evaluated head by head to bound memory.  `silu_dtype`: SiLU(V1)
    rounded to that dtype first, as the reference's kernel front-end does (oracle.gated)."""
    q, k1, k2, v1, v2, do = (t.float() for t in inputs)
    kw = dict(zip(("k1_window", "k2_window", "kk_left", "kk_right"), windows))
    if silu_dtype is not None:
        kw["silu_dtype"] = silu_dtype
    B, H, T, D = q.shape
    z = torch.empty_like(q)
    lse = torch.empty(B, H, T)
    grads = [torch.empty_like(q) for _ in range(5)]
    for b in range(B):
        for h in range(H):
            zz, ll, gg = orc.tdp_forward_backward(*(t[b, h] for t in (q, k1, k2, v1, v2, do)), alpha, causal, **kw)
            z[b, h], lse[b, h] = zz, ll
            for g, x in zip(grads, gg):
                g[b, h] = x
    return z, lse, grads


def oracle_dps(inputs, alpha, causal, k_diff, factorised=False):
    q, k1, k2, v1, v2, do = (t.float() for t in inputs)
    B, H, T, D = q.shape
    z = torch.empty_like(q)
    lse = torch.empty(B, H, T)
    grads = [torch.empty_like(q) for _ in range(5)]
    for b in range(B):
        for h in range(H):
            zz, ll, gg = orc.dps_forward_backward(*(t[b, h] for t in (q, k1, k2, v1, v2, do)), alpha, causal,
                                                  k_diff=k_diff, factorised=factorised)
            z[b, h], lse[b, h] = zz, ll
            for g, x in zip(grads, gg):
                g[b, h] = x
    return z, lse, grads


def run_tdp(inputs, alpha, causal, windows=(None,) * 4, backward=True, device="cuda", flags=0):
    from flash_trittention.triple_dot_product.flash_trittention import FlashTrittention, flash_trittention

    if flags:
        fn = FlashTrittention.with_flags(flags)
        flash_trittention = lambda q, k1, k2, v1, v2, softmax_scale, k1_window, k2_window, kk_left, kk_right, causal: \
            fn.apply(q, k1, k2, v1, v2, softmax_scale, kk_left, kk_right, k1_window, k2_window, causal, False)
    return _run_tdp(flash_trittention, inputs, alpha, causal, windows, backward, device)


def _run_tdp(flash_trittention, inputs, alpha, causal, windows, backward, device):

    q, k1, k2, v1, v2, do = (t.to(device) for t in inputs)
    leaves = [t.detach().clone().requires_grad_(backward) for t in (q, k1, k2, v1, v2)]
    out = flash_trittention(*leaves, softmax_scale=alpha, k1_window=windows[0], k2_window=windows[1],
                            kk_left=windows[2], kk_right=windows[3], causal=causal)
    grads = None
    if backward:
        out.backward(do)
        grads = [t.grad.float().cpu() for t in leaves]
    torch.cuda.synchronize()
    return out.detach().float().cpu(), grads


def run_dps(inputs, alpha, causal, k_diff, backward=True, device="cuda", flags=0):
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTritonFunction

    return _run_dps(inputs, alpha, causal, k_diff, backward, device, TrittentionTritonFunction.with_flags(flags))


def _run_dps(inputs, alpha, causal, k_diff, backward, device, function):
    q, k1, k2, v1, v2, do = (t.to(device) for t in inputs)
    leaves = [t.detach().clone().requires_grad_(backward) for t in (q, k1, k2, v1, v2)]
    out, m = function.apply(*leaves, causal, alpha, k_diff)
    grads = None
    if backward:
        out.backward(do)
        grads = [t.grad.float().cpu() for t in leaves]
    torch.cuda.synchronize()
    return out.detach().float().cpu(), m.detach().cpu(), grads


def assert_close(name, got, want, rtol, atol):
    torch.testing.assert_close(got, want, rtol=rtol, atol=atol, msg=lambda m: f"{name}: {m}")


def rel_err(got, want):
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def assert_mostly_close(name, got, want, rtol, atol, outlier_frac=0.0, outlier_scale=1.0):
    """assert_close that also prints the worst |err| / tol of the comparison.  By default every element must be
    within tolerance.  `outlier_frac` / `outlier_scale` let a stated fraction of the elements reach a stated
    multiple of the tolerance: used only where the comparison is not the parity bar itself (the library's MFMA
    kernels against its own fp32 kernels under scores scaled by 3) or where a single element of a very large
    tensor sits on the edge of the 16-bit bar; each such call says why."""
    err = (got - want).abs()
    tol = atol + rtol * want.abs()
    bad = err > tol
    worst = (err / tol).max().item() if err.numel() else 0.0
    print(f"    {name}: worst |err|/tol = {worst:.2f}, {int(bad.sum())} of {bad.numel()} beyond tol", flush=True)
    assert bad.float().mean().item() <= outlier_frac, f"{name}: {bad.sum().item()} of {bad.numel()} outside tolerance"
    assert (err <= outlier_scale * tol).all(), f"{name}: max error {err.max().item()}"


def check_offsets_beyond_32_bits(variant, B, H, T, D, windows=(None,) * 4, rtol=5e-2, atol=2e-2):
    """Forward and backward on bf16 tensors of more than 2^31 elements (inputs drawn on the device), checked
    against the oracle on the first head, the heads either side of element 2^31 and the last head."""
    import math

    from flash_trittention import TrittentionTriton, flash_trittention

    assert B * H * T * D > 2**31
    gen = torch.Generator(device="cuda").manual_seed(1)
    draw = lambda: torch.randn(B, H, T, D, device="cuda", dtype=torch.bfloat16, generator=gen)
    leaves = [draw().requires_grad_(True) for _ in range(5)]
    do = draw()
    alpha = 1 / math.sqrt(D)
    kw = dict(zip(("k1_window", "k2_window", "kk_left", "kk_right"), windows))
    if variant == "tdp":
        out = flash_trittention(*leaves, softmax_scale=alpha, causal=True, **kw)
    else:
        out, _ = TrittentionTriton(causal=True, softmax_scale=alpha, k_diff=T)(*leaves)
    out.backward(do)
    torch.cuda.synchronize()
    edge = 2**31 // (T * D)  # the head that holds element 2^31
    try:
        for hd in sorted({0, edge - 1, edge, edge + 1, B * H - 1}):
            b, h = divmod(hd, H)
            ins = [t.detach()[b, h].float().cpu() for t in leaves] + [do[b, h].float().cpu()]
            if variant == "tdp":
                z, _, grads = orc.tdp_forward_backward_chunked(*ins, alpha, True, q_chunk=128, **kw)
            else:
                z, _, grads = orc.dps_forward_backward(*ins, alpha, True, k_diff=T, factorised=True)
            assert_close(f"out[{hd}]", out.detach()[b, h].float().cpu(), z, rtol=rtol, atol=atol)
            for name, leaf, want in zip(NAMES, leaves, grads):
                # 512 x 128 elements per head and gradient at the edge of the 16-bit bar: one element in 10^4 may
                # reach 1.5 times the tolerance (seen: one of 65536 at 1.07)
                assert_mostly_close(f"{name}[{hd}]", leaf.grad[b, h].float().cpu(), want, rtol=rtol, atol=atol,
                                    outlier_frac=1e-4, outlier_scale=1.5)
    finally:
        del leaves, do, out
        torch.cuda.empty_cache()
