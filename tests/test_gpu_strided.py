"""Strided [B,H,T,D] views at the C ABI (tritt_*_strided): a projection layer's [B,T,H,D] output transposed, slices of
one fused [B,T,5,H,D] tensor, mixed layouts.  The reference accepts such views and copies them
(triple_dot_product/flash_trittention.py:64-68; its test: tests/test_dot_product_sum.py:121-134); here the 16-bit
matrix-core kernels read them where they lie and the other paths gather them inside the library's workspace.

Every case is held to two bars: the oracle at the dtype's tolerance, and the dense call on `.contiguous()` copies of
the same views bit for bit (the same kernels see the same numbers)."""
import ctypes
import math

import pytest
import torch

from oracle import trittention_oracle as orc
from tests import util

pytestmark = pytest.mark.gpu

LOWP = dict(rtol=5e-2, atol=2e-2)
FP32 = dict(rtol=2e-3, atol=2e-4)


def fused_views(B, H, T, D, dtype, seed):
    """q, k1, k2, v1, v2 as slices of one [B,T,5,H,D] tensor, each seen as [B,H,T,D] (strides 5HDT, D, 5HD, 1)."""
    g = torch.Generator().manual_seed(seed)
    fused = torch.randn(B, T, 5, H, D, generator=g).to(dtype).cuda()
    return [fused[:, :, i].transpose(1, 2) for i in range(5)], fused


def bthd_view(B, H, T, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, T, H, D, generator=g).to(dtype).cuda().transpose(1, 2)


def dense_inputs(views, d_o):
    return [t.detach().contiguous().cpu() for t in (*views, d_o)]


@pytest.mark.parametrize("shape,dtype,windows,causal", [
    ((2, 4, 256, 64), torch.bfloat16, (None,) * 4, True),
    ((1, 3, 203, 32), torch.bfloat16, (None,) * 4, True),
    ((1, 2, 160, 128), torch.float16, (None,) * 4, True),
    ((2, 2, 300, 64), torch.bfloat16, (100, 64, 33, 16), True),   # windowed streaming kernel
    ((2, 2, 300, 64), torch.bfloat16, (24, 22, None, None), True),  # band-resident kernel
    ((1, 2, 96, 32), torch.float32, (None,) * 4, True),           # fp32 tensors: gathered, then the dense kernels
    ((1, 2, 64, 16), torch.bfloat16, (None,) * 4, True),          # no matrix-core kernel at D = 16: gathered
    ((2, 6, 64, 64), torch.bfloat16, (None,) * 4, False),         # no mask; twelve slices: one whole group of eight and four over
    ((1, 5, 257, 128), torch.float16, (None,) * 4, False),
    ((1, 3, 64, 128), torch.bfloat16, (40, 24, 300, 0), True),    # band-resident kernel at D = 128
    ((1, 1, 100, 128), torch.float16, (None,) * 4, True),         # one batch, one head: both strides of extent-1 dimensions
])
def test_triple_dot_on_slices_of_a_fused_projection(shape, dtype, windows, causal):
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    print(f"case strided triple-dot {shape} {dtype} {windows} causal={causal}", flush=True)
    B, H, T, D = shape
    views, _ = fused_views(B, H, T, D, dtype, seed=T)
    assert not any(v.is_contiguous() for v in views)
    d_o = bthd_view(B, H, T, D, dtype, seed=T + 1)
    alpha = 1 / math.sqrt(D)
    kw = dict(softmax_scale=alpha, k1_window=windows[0], k2_window=windows[1], kk_left=windows[2], kk_right=windows[3],
              causal=causal)

    def run(tensors, grad):
        leaves = [t.detach().requires_grad_(True) for t in tensors]
        out = flash_trittention(*leaves, **kw)
        out.backward(grad)
        return out.detach(), [t.grad for t in leaves]

    out_s, g_s = run(views, d_o)
    out_d, g_d = run([v.contiguous() for v in views], d_o.contiguous())
    torch.cuda.synchronize()
    assert out_s.is_contiguous() and all(g.shape == (B, H, T, D) for g in g_s)
    assert torch.equal(out_s, out_d)
    for name, a, b in zip(util.NAMES, g_s, g_d):
        assert torch.equal(a, b), name

    inputs = dense_inputs(views, d_o)
    z, _, grads = util.oracle_tdp(inputs, alpha, causal, windows)
    tol = FP32 if dtype == torch.float32 else LOWP
    util.assert_mostly_close("out", out_s.float().cpu(), z, **tol)
    for name, a, b in zip(util.NAMES, g_s, grads):
        util.assert_mostly_close(name, a.float().cpu(), b, **tol)


@pytest.mark.parametrize("shape,dtype,causal", [((2, 4, 192, 64), torch.bfloat16, True), ((1, 2, 100, 32), torch.float16, True),
                                                ((2, 2, 64, 32), torch.float32, True), ((1, 2, 130, 128), torch.bfloat16, True),
                                                ((2, 6, 257, 64), torch.float16, False), ((1, 1, 257, 64), torch.float16, True)])
def test_dot_product_sum_on_transposed_projections(shape, dtype, causal):
    """All five inputs and dO as [B,T,H,D] tensors transposed (the layout tests/test_dot_product_sum.py:121-134 of the
    reference feeds for K1 and K2)."""
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTriton

    print(f"case strided dot-product-sum {shape} {dtype} causal={causal}", flush=True)
    B, H, T, D = shape
    views = [bthd_view(B, H, T, D, dtype, seed=10 * T + i) for i in range(5)]
    d_o = bthd_view(B, H, T, D, dtype, seed=10 * T + 5)
    module = TrittentionTriton(causal=causal, softmax_scale=1 / 8, k_diff=T // 2)

    def run(tensors, grad):
        leaves = [t.detach().requires_grad_(True) for t in tensors]
        out, m = module(*leaves)
        out.backward(grad)
        return out.detach(), m.detach(), [t.grad for t in leaves]

    out_s, m_s, g_s = run(views, d_o)
    out_d, m_d, g_d = run([v.contiguous() for v in views], d_o.contiguous())
    torch.cuda.synchronize()
    assert torch.equal(out_s, out_d) and torch.equal(m_s, m_d)
    for name, a, b in zip(util.NAMES, g_s, g_d):
        assert torch.equal(a, b), name
    z, _, grads = util.oracle_dps(dense_inputs(views, d_o), 1 / 8, causal, T // 2)
    tol = FP32 if dtype == torch.float32 else LOWP
    util.assert_mostly_close("out", out_s.float().cpu(), z, **tol)
    for name, a, b in zip(util.NAMES, g_s, grads):
        util.assert_mostly_close(name, a.float().cpu(), b, **tol)


def test_triple_dot_forward_reads_the_views_in_place():
    """The 16-bit matrix-core forward takes five slices of a fused tensor without a copy: its workspace is the dense
    call's, and the peak of device memory over the call is the outputs plus that workspace."""
    from flash_trittention import _lib, _ops

    B, H, T, D = 2, 8, 512, 64
    views, fused = fused_views(B, H, T, D, torch.bfloat16, seed=3)
    lay = _lib.layouts(views)
    assert lay is not None and all(_lib.viewable(v) for v in views)
    args = (B, H, T, D, _lib.TRITT_BF16, 1, T, T, T, T, 0)
    plain = _lib.lib().tritt_tdp_fwd_workspace_bytes(*args)
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, lay) == (plain + 255) // 256 * 256
    # four equal layouts and a dense V1 need no copy; nor do tensors that each have a layout of their own (K2 from
    # another projection, a dense Q): the kernel's second instantiation takes a layout per tensor
    mixed = [views[0], views[1], views[2], views[3].contiguous(), views[4]]
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, _lib.layouts(mixed)) == (plain + 255) // 256 * 256
    odd = [views[0].contiguous(), views[1], bthd_view(B, H, T, D, torch.bfloat16, 4), views[3], views[4].contiguous()]
    n_bytes = B * H * T * D * 2
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, _lib.layouts(odd)) == (plain + 255) // 256 * 256
    o_odd, lse_odd = _ops.tdp_fwd_impl(*odd, 1 / 8, True, T, T, T, T, 0)
    o_ref, lse_ref = _ops.tdp_fwd_impl(*(t.contiguous() for t in odd), 1 / 8, True, T, T, T, T, 0)
    assert torch.equal(o_odd, o_ref) and torch.equal(lse_odd, lse_ref)
    # a view that is a broadcast along t is gathered (its row stride of 0 would read as "dense" in the launch arguments)
    flat = [views[0], views[1], views[2], views[3], views[4][:, :, :1].expand(B, H, T, D)]
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, _lib.layouts(flat)) == \
        (plain + 255) // 256 * 256 + 5 * n_bytes
    o_flat, lse_flat = _ops.tdp_fwd_impl(*flat, 1 / 8, True, T, T, T, T, 0)
    o_ref, lse_ref = _ops.tdp_fwd_impl(*(t.contiguous() for t in flat), 1 / 8, True, T, T, T, T, 0)
    assert torch.equal(o_flat, o_ref) and torch.equal(lse_flat, lse_ref)

    _ops.tdp_fwd_impl(*views, 1 / 8, True, T, T, T, T, 0)  # first call: kernel attributes, allocator pools
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    o, lse = _ops.tdp_fwd_impl(*views, 1 / 8, True, T, T, T, T, 0)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    outputs = o.numel() * 2 + lse.numel() * 4
    assert grown <= outputs + plain + 4096, (grown, outputs, plain)  # one input copy would add n_bytes = 1 MiB
    assert grown < outputs + plain + n_bytes // 2
    o_d, lse_d = _ops.tdp_fwd_impl(*(v.contiguous() for v in views), 1 / 8, True, T, T, T, T, 0)
    assert torch.equal(o, o_d) and torch.equal(lse, lse_d)
    # V1 on a layout of its own, either way round (its pass takes its own strides and head count)
    o_m, lse_m = _ops.tdp_fwd_impl(*mixed, 1 / 8, True, T, T, T, T, 0)
    assert torch.equal(o_m, o_d) and torch.equal(lse_m, lse_d)
    only_v1 = [v.contiguous() for v in views]
    only_v1[3] = views[3]
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, _lib.layouts(only_v1)) == (plain + 255) // 256 * 256
    o_v, lse_v = _ops.tdp_fwd_impl(*only_v1, 1 / 8, True, T, T, T, T, 0)
    assert torch.equal(o_v, o_d) and torch.equal(lse_v, lse_d)
    del fused


@pytest.mark.parametrize("shape,windows,flags", [((2, 3, 300, 64), (None,) * 4, 0), ((1, 5, 200, 128), (None,) * 4, 0),
                                                 ((2, 2, 300, 64), (100, 64, 33, 16), 0), ((2, 2, 300, 64), (24, 22, 300, 300), 0),
                                                 ((1, 3, 130, 32), (None,) * 4, 0), ((1, 4, 200, 64), (None,) * 4, 8)])
def test_triple_dot_forward_with_a_layout_per_tensor(shape, windows, flags):
    """Q dense, K1 and V2 slices of a fused tensor, K2 a transposed projection, V1 a slice: the forward's second
    instantiation reads each where it lies (streaming, banded, band-resident and split-operand kernels, three head
    dimensions): the dense call's workspace, bitwise the dense call's results."""
    from flash_trittention import _lib, _ops

    print(f"case strided triple-dot forward, a layout per tensor {shape} {windows} flags={flags}", flush=True)
    B, H, T, D = shape
    fused, keep = fused_views(B, H, T, D, torch.bfloat16, seed=51)
    tensors = [fused[0].contiguous(), fused[1], bthd_view(B, H, T, D, torch.bfloat16, 52), fused[3], fused[4]]
    w = [T if x is None else x for x in windows]
    args = (B, H, T, D, _lib.TRITT_BF16, 1, *w, flags)
    plain = _lib.lib().tritt_tdp_fwd_workspace_bytes(*args)
    assert _lib.lib().tritt_tdp_fwd_strided_workspace_bytes(*args, _lib.layouts(tensors)) == (plain + 255) // 256 * 256
    o, lse = _ops.tdp_fwd_impl(*tensors, 1 / 8, True, *w, flags)
    o_d, lse_d = _ops.tdp_fwd_impl(*(t.contiguous() for t in tensors), 1 / 8, True, *w, flags)
    assert torch.equal(o, o_d) and torch.equal(lse, lse_d)
    del keep


@pytest.mark.parametrize("shape,windows,flags", [((2, 8, 512, 64), (None,) * 4, 0), ((1, 4, 384, 128), (None,) * 4, 0),
                                                 ((2, 4, 320, 64), (100, 64, 33, 16), 0), ((1, 4, 256, 32), (None,) * 4, 0),
                                                 ((1, 4, 200, 64), (None,) * 4, 8)])
def test_triple_dot_backward_reads_the_views_in_place(shape, windows, flags):
    """The 16-bit matrix-core backward takes slices of a fused projection and a transposed dO without a copy: its
    workspace is the dense call's, the peak of device memory over the call is the gradients plus that workspace, and
    every gradient is bitwise what the dense call returns (the D = 64 kernel, the 16-query kernel at D = 128, the banded
    kernels, D = 32, split operands; the first query tile runs on the fp32 kernels, which take the strides too)."""
    from flash_trittention import _lib, _ops

    print(f"case strided triple-dot backward in place {shape} {windows} flags={flags}", flush=True)
    B, H, T, D = shape
    views, fused = fused_views(B, H, T, D, torch.bfloat16, seed=41)
    d_o = bthd_view(B, H, T, D, torch.bfloat16, seed=42)
    w = [T if x is None else x for x in windows]
    lay, lay_do = _lib.layouts(views), _lib.layouts([d_o])
    args = (B, H, T, D, _lib.TRITT_BF16, 1, *w, flags)
    api = _lib.lib()
    plain = api.tritt_tdp_bwd_workspace_bytes(*args)
    assert api.tritt_tdp_bwd_strided_workspace_bytes(*args, lay, lay_do) == (plain + 255) // 256 * 256
    n_bytes = B * H * T * D * 2
    o, lse = _ops.tdp_fwd_impl(*views, 1 / 8, True, *w, flags)
    _ops.tdp_bwd_impl(*views, o, lse, d_o, 1 / 8, True, *w, flags, 31)  # first call: kernel attributes, allocator pools
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    grads = _ops.tdp_bwd_impl(*views, o, lse, d_o, 1 / 8, True, *w, flags, 31)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    # the allocator rounds a large block up to 2 MiB; six gathered views would add 6 n_bytes
    assert grown < 5 * n_bytes + plain + (2 << 20) + n_bytes, (grown, plain, n_bytes)
    dense = [v.contiguous() for v in views]
    o_d, lse_d = _ops.tdp_fwd_impl(*dense, 1 / 8, True, *w, flags)
    assert torch.equal(o, o_d) and torch.equal(lse, lse_d)
    grads_d = _ops.tdp_bwd_impl(*dense, o_d, lse_d, d_o.contiguous(), 1 / 8, True, *w, flags, 31)
    for name, a, b in zip(util.NAMES, grads, grads_d):
        assert torch.equal(a, b), name
    # a dense dO with strided inputs, and the other way round
    for ins, g in ((views, d_o.contiguous()), (dense, d_o)):
        mixed = _ops.tdp_bwd_impl(*ins, o, lse, g, 1 / 8, True, *w, flags, 31)
        for name, a, b in zip(util.NAMES, mixed, grads_d):
            assert torch.equal(a, b), name
    del fused


def test_dot_product_sum_reads_the_views_in_place():
    """The 16-bit matrix-core kernels of dot-product-sum take [B,T,H,D] tensors transposed, and dO likewise, without a
    copy: forward and backward ask for the dense calls' workspaces, and the peak of device memory over each call is
    its outputs plus that workspace."""
    from flash_trittention import _lib, _ops

    B, H, T, D = 4, 8, 1024, 64
    views = [bthd_view(B, H, T, D, torch.bfloat16, seed=20 + i) for i in range(5)]
    d_o = bthd_view(B, H, T, D, torch.bfloat16, seed=26)
    lay, lay_do = _lib.layouts(views), _lib.layouts([d_o])
    api = _lib.lib()
    args = (B, H, T, D, _lib.TRITT_BF16, 0)
    plain_f, plain_b = api.tritt_dps_fwd_workspace_bytes(*args), api.tritt_dps_bwd_workspace_bytes(*args)
    assert api.tritt_dps_fwd_strided_workspace_bytes(*args, lay) == (plain_f + 255) // 256 * 256
    assert api.tritt_dps_bwd_strided_workspace_bytes(*args, lay, lay_do) == (plain_b + 255) // 256 * 256
    n_bytes = B * H * T * D * 2

    o, m = _ops.dps_fwd_impl(*views, 1 / 8, True, T, 0)  # first calls: kernel attributes, allocator pools
    _ops.dps_bwd_impl(*views, o, m, d_o, 1 / 8, True, T, 0)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    o, m = _ops.dps_fwd_impl(*views, 1 / 8, True, T, 0)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    slack = 2 << 20  # the allocator rounds a large block up to 2 MiB; one copy of one view would add n_bytes = 4 MiB
    assert grown < o.numel() * 2 + m.numel() * 4 + plain_f + slack, (grown, plain_f)
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    grads = _ops.dps_bwd_impl(*views, o, m, d_o, 1 / 8, True, T, 0)
    torch.cuda.synchronize()
    grown = torch.cuda.max_memory_allocated() - before
    assert grown < 5 * n_bytes + plain_b + slack, (grown, plain_b)
    dense = [v.contiguous() for v in views]
    o_d, m_d = _ops.dps_fwd_impl(*dense, 1 / 8, True, T, 0)
    grads_d = _ops.dps_bwd_impl(*dense, o_d, m_d, d_o.contiguous(), 1 / 8, True, T, 0)
    assert torch.equal(o, o_d) and torch.equal(m, m_d)
    for name, a, b in zip(util.NAMES, grads, grads_d):
        assert torch.equal(a, b), name
    # broadcast views (a stride of zero) are read in place as well
    one = torch.randn(1, 1, T, D, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    shared = [one.expand(B, H, T, D) for _ in range(5)]
    o_b, m_b = _ops.dps_fwd_impl(*shared, 1 / 8, True, T, 0)
    o_c, m_c = _ops.dps_fwd_impl(*(t.contiguous() for t in shared), 1 / 8, True, T, 0)
    assert torch.equal(o_b, o_c) and torch.equal(m_b, m_c)


def test_split_operands_and_static_layout_cases():
    """convert_to_float32 (split operands) on strided views; extent-1 dimensions with arbitrary strides; a broadcast
    (stride 0) head dimension."""
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    B, H, T, D = 1, 2, 128, 64
    views, _ = fused_views(B, H, T, D, torch.bfloat16, seed=9)
    a = flash_trittention(*views, softmax_scale=1 / 8, k1_window=None, k2_window=None, kk_left=None, kk_right=None,
                          causal=True, convert_to_float32=True)
    b = flash_trittention(*(v.contiguous() for v in views), softmax_scale=1 / 8, k1_window=None, k2_window=None,
                          kk_left=None, kk_right=None, causal=True, convert_to_float32=True)
    assert torch.equal(a, b)
    # one head broadcast to two: stride_h = 0
    base = [torch.randn(1, 1, T, D, generator=torch.Generator().manual_seed(i)).bfloat16().cuda() for i in range(5)]
    wide = [t.expand(1, 2, T, D) for t in base]
    a = flash_trittention(*wide, softmax_scale=1 / 8, k1_window=None, k2_window=None, kk_left=None, kk_right=None)
    b = flash_trittention(*(t.contiguous() for t in wide), softmax_scale=1 / 8, k1_window=None, k2_window=None,
                          kk_left=None, kk_right=None)
    assert torch.equal(a, b) and torch.equal(a[:, 0], a[:, 1])


def test_layouts_the_library_refuses():
    """Strides that would break the 16-byte pieces are an error at the C ABI (the Python front copies such views
    first, as the reference copies every view)."""
    from flash_trittention import _lib
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    B, H, T, D = 1, 2, 64, 32
    g = torch.Generator().manual_seed(0)
    big = torch.randn(B, H, T, D + 4, generator=g).bfloat16().cuda()
    odd = big[..., :D]  # row stride 36 elements: not a multiple of 16 bytes
    assert not _lib.viewable(odd)
    dense = [torch.randn(B, H, T, D, generator=g).bfloat16().cuda() for _ in range(4)]
    out = flash_trittention(odd, *dense)
    assert torch.equal(out, flash_trittention(odd.contiguous(), *dense))

    lay = (_lib.Layout * 5)()
    for slot in lay:
        slot.stride_b, slot.stride_h, slot.stride_t = H * T * D, T * D, D
    lay[0].stride_t = D + 4
    o = torch.empty(B, H, T, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, T, dtype=torch.float32, device="cuda")
    ws = torch.empty(1 << 22, dtype=torch.uint8, device="cuda")
    ptrs = [_lib.ptr(t) for t in (odd, *dense)]
    st = _lib.lib().tritt_tdp_fwd_strided(*ptrs, lay, _lib.ptr(o), _lib.ptr(lse), B, H, T, D, _lib.TRITT_BF16, 0.125, 1,
                                          T, T, T, T, _lib.ptr(ws), ws.numel(), 0, _lib.stream_ptr(o.device))
    assert st == -1  # TRITT_ERR_INVALID
    lay[0].stride_t = -D
    st = _lib.lib().tritt_dps_fwd_strided(*ptrs, lay, _lib.ptr(o), _lib.ptr(lse), B, H, T, D, _lib.TRITT_BF16, 0.125, 1,
                                          T, _lib.ptr(ws), ws.numel(), 0, _lib.stream_ptr(o.device))
    assert st == -1
    # too small a workspace: for the gathered copy of the fp32 path, for the call itself on the matrix-core path
    lay[0].stride_t = 2 * D
    wide = torch.randn(B, H, T, 2 * D, generator=g).bfloat16().cuda()
    ptrs[0] = _lib.ptr(wide)
    for flags, copies in ((_lib.FLAG_FORCE_GENERIC, 1), (0, 0)):
        need = _lib.lib().tritt_dps_fwd_strided_workspace_bytes(B, H, T, D, _lib.TRITT_BF16, flags, lay)
        plain = _lib.lib().tritt_dps_fwd_workspace_bytes(B, H, T, D, _lib.TRITT_BF16, flags)
        assert need == (plain + 255) // 256 * 256 + copies * B * H * T * D * 2
        st = _lib.lib().tritt_dps_fwd_strided(*ptrs, lay, _lib.ptr(o), _lib.ptr(lse), B, H, T, D, _lib.TRITT_BF16, 0.125,
                                              1, T, _lib.ptr(ws), need - 1, flags, _lib.stream_ptr(o.device))
        assert st == -3  # TRITT_ERR_WORKSPACE
        st = _lib.lib().tritt_dps_fwd_strided(*ptrs, lay, _lib.ptr(o), _lib.ptr(lse), B, H, T, D, _lib.TRITT_BF16, 0.125,
                                              1, T, _lib.ptr(ws), need, flags, _lib.stream_ptr(o.device))
        assert st == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("variant", ["tdp", "dps"])
@pytest.mark.parametrize("shape,dtype", [((2, 4, 256, 64), torch.bfloat16), ((1, 3, 150, 128), torch.float16),
                                         ((2, 2, 100, 32), torch.bfloat16), ((1, 2, 96, 32), torch.float32)])
@pytest.mark.parametrize("strided", ["dO", "inputs"])
def test_only_one_side_is_strided(variant, shape, dtype, strided):
    """The layout of a model's backward: dense q, k1, k2, v1, v2 and an incoming gradient that is a [B,T,H,D] tensor
    transposed (what autograd hands back when the output is transposed for the next projection), and the reverse
    (transposed projections in, a dense gradient).  The C ABI then gets a null layout array for the dense side.  All
    five gradients bitwise those of the call on dense copies."""
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTriton

    B, H, T, D = shape
    print(f"case one side strided: {variant} {shape} {dtype} strided={strided}", flush=True)
    if strided == "inputs":
        ins = [bthd_view(B, H, T, D, dtype, seed=20 + i) for i in range(5)]
        d_o = torch.randn(B, H, T, D, generator=torch.Generator().manual_seed(7)).to(dtype).cuda()
    else:
        g = torch.Generator().manual_seed(8)
        ins = [torch.randn(B, H, T, D, generator=g).to(dtype).cuda() for _ in range(5)]
        d_o = bthd_view(B, H, T, D, dtype, seed=9)
    assert d_o.is_contiguous() == (strided == "inputs")
    alpha = 1 / math.sqrt(D)
    if variant == "tdp":
        fn = lambda *t: flash_trittention(*t, softmax_scale=alpha, k1_window=None, k2_window=None, kk_left=None,
                                          kk_right=None, causal=True)
    else:
        mod = TrittentionTriton(causal=True, softmax_scale=alpha, k_diff=T)
        fn = lambda *t: mod(*t)[0]

    def grads(tensors, go):
        leaves = [t.detach().clone(memory_format=torch.preserve_format).requires_grad_(True) for t in tensors]
        # clone() of a transposed view keeps its strides: the leaves are laid out like the tensors handed in
        assert all(a.stride() == b.stride() for a, b in zip(leaves, tensors))
        out = fn(*leaves)
        out.backward(go)
        return [out.detach()] + [t.grad for t in leaves]

    got = grads(ins, d_o)
    want = grads([t.contiguous() for t in ins], d_o.contiguous())
    for name, a, b in zip(("out",) + tuple(util.NAMES), got, want):
        assert torch.equal(a.contiguous(), b.contiguous()), name
    if variant == "tdp":
        z, _, ref = util.oracle_tdp(dense_inputs(ins, d_o), alpha, True)
    else:
        z, _, ref = util.oracle_dps(dense_inputs(ins, d_o), alpha, True, T)
    tol = FP32 if dtype == torch.float32 else LOWP
    util.assert_close("out", got[0].float().cpu(), z, **tol)
    for name, a, b in zip(util.NAMES, got[1:], ref):
        util.assert_close(name, a.float().cpu(), b, **tol)
