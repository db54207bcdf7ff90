"""GPU parity: triple-dot-product trittention (HIP, through the C ABI) vs the CPU oracle.

Tolerances: fp32 tensors 1e-4 relative (rtol 1e-4 with a small atol, and
max|err|/max|ref| <= 1e-4); bf16/fp16 tensors atol 2e-2 / rtol 5e-2 — the
bars the task states.  The case grid follows the reference's own tests
(tests/test_triple_dot_product.py:52-182)."""
import math

import pytest
import torch

from oracle import trittention_oracle as orc
from flash_trittention import _lib
from tests import util

pytestmark = pytest.mark.gpu

FP32 = dict(rtol=1e-4, atol=2e-5)
LOWP = dict(rtol=5e-2, atol=2e-2)


def check_all(inputs, alpha, causal, windows=(None,) * 4, tol=FP32, rel=1e-4):
    z, lse, grads = util.oracle_tdp(inputs, alpha, causal, windows)
    out, g = util.run_tdp(inputs, alpha, causal, windows)
    util.assert_close("out", out, z, **tol)
    assert util.rel_err(out, z) <= rel, util.rel_err(out, z)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_close(name, a, b, **tol)
        assert util.rel_err(a, b) <= rel, (name, util.rel_err(a, b))


@pytest.mark.parametrize("seq_len", [33, 64, 100])
@pytest.mark.parametrize("causal", [True, False])
def test_forward_and_backward_fp32(seq_len, causal):
    print(f"case fp32 T={seq_len} causal={causal}", flush=True)
    inputs = orc.make_inputs(2, 2, seq_len, 32, torch.float32, seed=seq_len)
    check_all(inputs, 1 / 8, causal)


@pytest.mark.parametrize("seq_len", [64, 100])
@pytest.mark.parametrize("windows", [(8, 8, 4, 4), (5, 3, 4, 1), (2, 70, 0, 3)])
def test_narrow_windows_causal(seq_len, windows):
    print(f"case windows T={seq_len} {windows}", flush=True)
    inputs = orc.make_inputs(2, 2, seq_len, 32, torch.float32, seed=7)
    check_all(inputs, 1 / 8, True, windows)


def test_config1_forward_fp32():
    """B=1 H=2 T=64 D=32 fp32, alpha = 1/sqrt(D), causal: output within 1e-4 relative."""
    inputs = orc.make_inputs(1, 2, 64, 32, torch.float32, seed=1)
    alpha = 1 / math.sqrt(32)
    z, lse, _ = util.oracle_tdp(inputs, alpha, True)
    out, _ = util.run_tdp(inputs, alpha, True, backward=False)
    util.assert_close("out", out, z, **FP32)
    assert util.rel_err(out, z) <= 1e-4


@pytest.mark.parametrize("D", [8, 16, 64, 128])
def test_head_dims_fp32(D):
    print(f"case fp32 D={D}", flush=True)
    inputs = orc.make_inputs(1, 2, 48, D, torch.float32, seed=D)
    check_all(inputs, 1 / math.sqrt(D), True)


def test_head_dim_8_bf16():
    """16-bit tensors with the smallest head dimension: computed by the fp32 kernels, held to the 16-bit bar."""
    inputs = orc.make_inputs(2, 3, 70, 8, torch.bfloat16, seed=8)
    alpha = 1 / math.sqrt(8)
    z, _, grads = util.oracle_tdp(inputs, alpha, True)
    out, g = util.run_tdp(inputs, alpha, True)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_close(name, a, b, **LOWP)


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("causal,windows", [(True, (None,) * 4), (False, (None,) * 4), (True, (100, 40, 24, 7)),
                                            (True, (3, 200, 0, 2))])
def test_fp32_tensors_on_the_matrix_cores(D, causal, windows, tune):
    """fp32 tensors on the fp32 MFMA kernels (enough query tiles for the launcher to pick them; ragged length):
    forward and all five gradients at the fp32 bar, and against the fp32 VALU kernels of the same library."""
    print(f"case fp32 mfma D={D} causal={causal} {windows}", flush=True)
    inputs = orc.make_inputs(2, 4, 250, D, torch.float32, seed=D + 3)
    alpha = 1 / math.sqrt(D)
    check_all(inputs, alpha, causal, windows)
    out, g = util.run_tdp(inputs, alpha, causal, windows)
    tune(_lib.TUNE_F32_VALU, 1)
    out_v, g_v = util.run_tdp(inputs, alpha, causal, windows)
    assert not torch.equal(out, out_v), "both runs took the same kernels"
    util.assert_close("out vs VALU kernels", out, out_v, **FP32)
    for name, a, b in zip(util.NAMES, g, g_v):
        util.assert_close(f"{name} vs VALU kernels", a, b, **FP32)


@pytest.mark.parametrize("causal", [True, False])
def test_fp32_head_dim_128_large_grid_on_the_matrix_cores(causal, tune):
    """D = 128 with enough query tiles that each is walked by one workgroup (dQ written by that workgroup, its running
    sum kept in LDS): against the fp32 VALU kernels of the same library, bitwise the same on a second run."""
    print(f"case fp32 mfma D=128 large grid causal={causal}", flush=True)
    inputs = orc.make_inputs(2, 4, 530, 128, torch.float32, seed=11)
    alpha = 1 / math.sqrt(128)
    out, g = util.run_tdp(inputs, alpha, causal)
    out2, g2 = util.run_tdp(inputs, alpha, causal)
    for name, a, b in zip(util.NAMES, g, g2):
        assert torch.equal(a, b), name
    tune(_lib.TUNE_F32_VALU, 1)
    out_v, g_v = util.run_tdp(inputs, alpha, causal)
    assert not torch.equal(out, out_v), "both runs took the same kernels"
    util.assert_close("out vs VALU kernels", out, out_v, **FP32)
    for name, a, b in zip(util.NAMES, g, g_v):
        util.assert_close(f"{name} vs VALU kernels", a, b, **FP32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_config2_lowp_forward_backward(dtype):
    """B=2 H=4 T=256 D=64, 16-bit tensors with fp32 accumulation, all five gradients."""
    print(f"case config2 {dtype}", flush=True)
    inputs = orc.make_inputs(2, 4, 256, 64, dtype, seed=2)
    check_all(inputs, 1 / 8, True, tol=LOWP, rel=2e-2)


def test_forward_fp16_loose():
    inputs = orc.make_inputs(2, 2, 64, 32, torch.float16, seed=3)
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True)
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False)
    util.assert_close("out", out, z, **LOWP)


def test_lse_matches_oracle():
    from flash_trittention.triple_dot_product.flash_trittention import FlashTrittention

    inputs = orc.make_inputs(1, 2, 40, 32, torch.float32, seed=4)
    z, lse, _ = util.oracle_tdp(inputs, 0.2, True)

    class Ctx:
        def save_for_backward(self, *t):
            self.saved = t

    ctx = Ctx()
    FlashTrittention.forward(ctx, *(t.cuda() for t in inputs[:5]), 0.2, None, None, None, None, True, False)
    util.assert_close("lse", ctx.saved[6].cpu(), lse, rtol=1e-5, atol=1e-5)


def test_reproducible(tune):
    """Every result is bitwise equal from run to run: the forward and (one workgroup per query tile) dQ have a
    single owner per element and a fixed summation order; dK1/dV1/dK2/dV2 of the MFMA path are summed over
    query tiles, and so is dQ when a small grid deals the rows of a tile out to several workgroups, in 64-bit
    fixed point with integer atomics, whose sum does not depend on the order of arrival.  The fp32 VALU path
    has one owner per element throughout."""
    inputs = orc.make_inputs(1, 2, 96, 64, torch.bfloat16, seed=5)
    tune(_lib.TUNE_BWD_SPLITS, 1)
    a = util.run_tdp(inputs, 1 / 8, True)
    b = util.run_tdp(inputs, 1 / 8, True)
    assert torch.equal(a[0], b[0])
    for i in range(5):
        assert torch.equal(a[1][i], b[1][i]), util.NAMES[i]
    tune(_lib.TUNE_BWD_SPLITS, 0)
    e = util.run_tdp(inputs, 1 / 8, True)  # this grid is small: rows split, dQ accumulated too
    f = util.run_tdp(inputs, 1 / 8, True)
    assert torch.equal(a[0], e[0])
    for i in range(5):
        assert torch.equal(e[1][i], f[1][i]), util.NAMES[i]
        util.assert_close(util.NAMES[i], a[1][i], e[1][i], rtol=1e-2, atol=1e-2)
    c = util.run_tdp(inputs, 1 / 8, True, flags=1)
    d = util.run_tdp(inputs, 1 / 8, True, flags=1)
    assert torch.equal(c[0], d[0])
    for x, y in zip(c[1], d[1]):
        assert torch.equal(x, y)


FLOAT_ATOMICS = _lib.FLAG_FLOAT_ATOMICS


@pytest.mark.parametrize("shape", [(2, 4, 256, 64), (4, 8, 1024, 64), (1, 3, 203, 128), (1, 3, 203, 32)])
def test_backward_is_bitwise_reproducible(shape):
    """The shares of the row gradients (and of a split dQ) are added as 64-bit fixed point with integer atomics,
    so two runs agree bit for bit in all five gradients whatever order the workgroups arrive in: BASELINE
    configs 2 (a small grid: rows split, dQ accumulated too) and 3, and the general kernel (D = 128, D = 32,
    ragged length).  With TRITT_FLAG_FLOAT_ATOMICS (fp32 atomics) the results differ from these by rounding."""
    print(f"case reproducible {shape}", flush=True)
    B, H, T, D = shape
    inputs = orc.make_inputs(B, H, T, D, torch.bfloat16, seed=T + D)
    alpha = 1 / math.sqrt(D)
    out_a, a = util.run_tdp(inputs, alpha, True)
    out_b, b = util.run_tdp(inputs, alpha, True)
    assert torch.equal(out_a, out_b)
    for name, x, y in zip(util.NAMES, a, b):
        assert torch.equal(x, y), name
    _, c = util.run_tdp(inputs, alpha, True, flags=FLOAT_ATOMICS)
    for name, x, y in zip(util.NAMES, a, c):
        util.assert_close(name, x, y, rtol=1e-2, atol=1e-2)


def test_float_atomics_flag_config2_against_oracle():
    inputs = orc.make_inputs(2, 4, 256, 64, torch.bfloat16, seed=2)
    z, lse, grads = util.oracle_tdp(inputs, 1 / 8, True)
    out, g = util.run_tdp(inputs, 1 / 8, True, flags=FLOAT_ATOMICS)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_close(name, a, b, **LOWP)
        assert util.rel_err(a, b) <= 2e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_only_the_requested_gradients_are_computed(dtype):
    """Inputs that do not require a gradient get none (a null pointer at the C ABI; launches that serve only
    unwanted gradients are skipped); the requested ones equal those of a run that asks for all five, bit for bit."""
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    inputs = [t.cuda() for t in orc.make_inputs(1, 2, 150, 64, dtype, seed=12)]
    kw = dict(softmax_scale=1 / 8, k1_window=None, k2_window=None, kk_left=None, kk_right=None, causal=True)
    full = [t.clone().requires_grad_(True) for t in inputs[:5]]
    flash_trittention(*full, **kw).backward(inputs[5])
    for wanted in ((0,), (1, 3), (2,), (4,), (0, 1), (3, 4)):
        leaves = [t.clone().requires_grad_(i in wanted) for i, t in enumerate(inputs[:5])]
        flash_trittention(*leaves, **kw).backward(inputs[5])
        for i, (a, b) in enumerate(zip(leaves, full)):
            if i in wanted:
                assert torch.equal(a.grad, b.grad), (wanted, util.NAMES[i])
            else:
                assert a.grad is None, (wanted, util.NAMES[i])


def test_non_contiguous_inputs():
    g = torch.Generator().manual_seed(11)
    q, v1, v2, do = (torch.randn(2, 4, 64, 32, generator=g) for _ in range(4))
    k1 = torch.randn(2, 64, 4, 32, generator=g).transpose(1, 2)
    k2 = torch.randn(2, 64, 4, 32, generator=g).transpose(1, 2)
    inputs = [q, k1, k2, v1, v2, do]
    z, _, grads = util.oracle_tdp([t.contiguous() for t in inputs], 1 / 8, True)
    out, g_ = util.run_tdp(inputs, 1 / 8, True)
    util.assert_close("out", out, z, **FP32)
    for name, a, b in zip(util.NAMES, g_, grads):
        util.assert_close(name, a, b, **FP32)


def test_rejects_mismatched_shapes():
    from flash_trittention import flash_trittention

    q, k1, k2, v1, v2, _ = (t.cuda() for t in orc.make_inputs(2, 2, 32, 32))
    with pytest.raises(ValueError):
        flash_trittention(q, k1, k2, v1, v2[:, :, :16, :].contiguous())
    with pytest.raises(ValueError):
        flash_trittention(q, k1, k2, v1, v2.half())


def test_rejects_non_pow2_head_dim():
    from flash_trittention import flash_trittention

    q, k1, k2, v1, v2, _ = (t.cuda() for t in orc.make_inputs(2, 2, 32, 24))
    with pytest.raises(ValueError):
        flash_trittention(q, k1, k2, v1, v2)


def test_input_precision_warns_and_is_ignored():
    from flash_trittention import flash_trittention

    q, k1, k2, v1, v2, _ = (t.cuda() for t in orc.make_inputs(1, 1, 16, 16))
    with pytest.warns(UserWarning):
        a = flash_trittention(q, k1, k2, v1, v2, k1_window=None, k2_window=None, kk_left=None, kk_right=None,
                              input_precision="ieee")
    b = flash_trittention(q, k1, k2, v1, v2, k1_window=None, k2_window=None, kk_left=None, kk_right=None)
    assert torch.equal(a, b)


# ---------------------------------------------------------------- MFMA kernels (16-bit tensors)
FORCE_GENERIC, FORCE_MFMA = 1, 2


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seq_len", [1, 16, 33, 100, 129, 256])
def test_mfma_forward_bf16(seq_len, causal, D):
    """The MFMA forward alone (FORCE_MFMA: no fallback), ragged lengths included."""
    print(f"case mfma fwd T={seq_len} causal={causal} D={D}", flush=True)
    inputs = orc.make_inputs(1, 3, seq_len, D, torch.bfloat16, seed=seq_len + D)
    alpha = 1 / math.sqrt(D)
    z, _, _ = util.oracle_tdp(inputs, alpha, causal)
    out, _ = util.run_tdp(inputs, alpha, causal, backward=False, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    # unmasked rows average ~T^2 terms: the outputs are small and the 16-bit rounding of P shows in max-relative terms
    assert util.rel_err(out, z) <= (3e-2 if D == 32 else 2e-2), util.rel_err(out, z)


WINDOWS = [(8, 8, 4, 4), (5, 3, 4, 1), (2, 70, 0, 3), (40, 100, 20, 7), (64, 64, 64, 64), (100, 10, 50, 0),
           (1, 1, 1, 1), (300, 300, 0, 0)]


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("windows", WINDOWS)
@pytest.mark.parametrize("seq_len", [33, 100, 300])
def test_mfma_forward_windows_bf16(seq_len, windows, D):
    """Windowed masks on the MFMA forward (banded k-tile / stage loops, element-wise masks)."""
    print(f"case mfma fwd windows T={seq_len} {windows} D={D}", flush=True)
    inputs = orc.make_inputs(1, 2, seq_len, D, torch.bfloat16, seed=seq_len + D + sum(windows))
    alpha = 1 / math.sqrt(D)
    z, _, _ = util.oracle_tdp(inputs, alpha, True, windows)
    out, _ = util.run_tdp(inputs, alpha, True, windows, backward=False, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    assert util.rel_err(out, z) <= 2e-2, util.rel_err(out, z)


@pytest.mark.parametrize("windows", [(40, 100, 20, 7), (5, 3, 4, 1), (100, 10, 50, 0)])
def test_mfma_forward_windows_large_logits(windows):
    """Scores spanning hundreds with windowed masks: the repeat sweep must cope with rows whose first
    valid key comes several steps into the sweep."""
    inputs = orc.make_inputs(1, 2, 200, 64, torch.bfloat16, seed=23)
    inputs[1] = (inputs[1].float() * 6).bfloat16()
    inputs[2] = (inputs[2].float() * 6).bfloat16()
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True, windows)
    out, _ = util.run_tdp(inputs, 1 / 8, True, windows, backward=False, flags=FORCE_MFMA)
    assert torch.isfinite(out).all()
    # same statistical bound as the unwindowed case below: 16-bit rounding of Q*K2 swaps near-tied winners
    err = (out - z).abs()
    assert (err > 5e-2).float().mean() < 0.01 and err.max() < 0.5, (err.max(), (err > 5e-2).float().mean())


def test_mfma_forward_fp16():
    inputs = orc.make_inputs(2, 2, 200, 64, torch.float16, seed=21)
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True)
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)


def test_mfma_forward_large_logits():
    """Scores spanning hundreds: the lazily raised reference maximum must keep everything finite."""
    inputs = orc.make_inputs(1, 2, 160, 64, torch.bfloat16, seed=22)
    inputs[1] = (inputs[1].float() * 6).bfloat16()
    inputs[2] = (inputs[2].float() * 6).bfloat16()
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True)
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)
    assert torch.isfinite(out).all()
    # with logits this large the softmax is nearly one-hot and the 16-bit rounding of Q*K2 can swap
    # near-tied winners (the reference's test notes the same), so bound the error statistically
    err = (out - z).abs()
    assert (err > 5e-2).float().mean() < 0.01 and err.max() < 0.5, (err.max(), (err > 5e-2).float().mean())


SPLIT = _lib.FLAG_SPLIT_OPERANDS


@pytest.mark.parametrize("windows", [(None,) * 4, (64, 100, 20, 30), (24, 22, None, None), (3, 200, 0, 2)])
@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (32, torch.bfloat16), (64, torch.float16), (128, torch.bfloat16)])
def test_large_logits_with_convert_to_float32_hold_the_16_bit_bar(windows, D, dtype):
    """convert_to_float32=True keeps the operands of the score products beyond 16-bit rounding, as the reference's
    flag does (triple_dot_product/flash_trittention.py:408, kernels/bwd_dq.py:197,219): D = 32 / 64 as hi + lo
    pairs on the 16-bit matrix-core kernels, D = 128 on the fp32 kernels.  Scores spanning hundreds, where the
    default path is held to a statistical bound, then meet the ordinary 16-bit tolerance element by element,
    forward and all five gradients.  The matrix-core kernels take SiLU(V1) rounded to the tensor dtype, as the
    reference's kernels do (flash_trittention.py:62); with nearly one-hot softmax rows that rounding alone moves
    dQ by several times the tolerance (every dP of a row shifts by 2^-9 |dP| independently, and K1 (.) K2 is 36
    times larger here), so those cases are compared with the oracle on the same rounded SiLU(V1)."""
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    print(f"case large logits, convert_to_float32: D={D} {dtype} {windows}", flush=True)
    inputs = orc.make_inputs(1, 2, 160, D, dtype, seed=22)
    scale = 6 if dtype == torch.bfloat16 else 4  # fp16: products of the scaled inputs stay inside half precision
    inputs[1] = (inputs[1].float() * scale).to(dtype)
    inputs[2] = (inputs[2].float() * scale).to(dtype)
    alpha = 1 / math.sqrt(D)
    z, _, grads = util.oracle_tdp(inputs, alpha, True, windows, silu_dtype=dtype if D != 128 else None)
    leaves = [t.cuda().requires_grad_(True) for t in inputs[:5]]
    out = flash_trittention(*leaves, softmax_scale=alpha, k1_window=windows[0], k2_window=windows[1], kk_left=windows[2],
                            kk_right=windows[3], causal=True, convert_to_float32=True)
    out.backward(inputs[5].cuda())
    err = (out.detach().float().cpu() - z).abs()
    assert err.max() < 5e-2, err.max()
    util.assert_mostly_close("out", out.detach().float().cpu(), z, **LOWP)
    for name, leaf, want in zip(util.NAMES, leaves, grads):
        util.assert_mostly_close(name, leaf.grad.float().cpu(), want, **LOWP)


@pytest.mark.parametrize("shape,windows", [((2, 4, 256, 64), (None,) * 4), ((1, 3, 203, 32), (None,) * 4),
                                           ((1, 2, 449, 64), (100, 64, 33, 16)), ((2, 2, 130, 64), (3, 200, 0, 2)),
                                           ((1, 5, 64, 32), (8, 8, 4, 4))])
@pytest.mark.parametrize("causal", [True, False])
def test_split_operands_through_the_c_abi(shape, windows, causal):
    """TRITT_FLAG_SPLIT_OPERANDS on ordinary inputs: every result at the 16-bit bar against the oracle, the output
    bitwise what the flag-less call stores where the two agree on the rounding (most elements), and the second
    tensor behind `o` the rounding residual of the first."""
    from flash_trittention import _ops

    print(f"case split operands {shape} {windows} causal={causal}", flush=True)
    B, H, T, D = shape
    inputs = orc.make_inputs(B, H, T, D, torch.bfloat16, seed=T)
    alpha = 1 / math.sqrt(D)
    z, _, grads = util.oracle_tdp(inputs, alpha, causal, windows)
    out, g = util.run_tdp(inputs, alpha, causal, windows, flags=SPLIT)
    util.assert_mostly_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
    dev = [t.cuda() for t in inputs[:5]]
    w = [T if x is None else x for x in windows]
    o2, lse = _ops.tdp_fwd_impl(*dev, alpha, causal, *w, SPLIT)
    assert o2.shape == (2, B, H, T, D)
    # the residual is what rounding to 16 bit removed: below half an ulp of the stored value, and adding it back
    # moves the result towards the fp32 oracle on average
    assert (o2[1].float().abs() <= o2[0].float().abs() * 2.0 ** -8 + 1e-30).all()
    full = (o2[0].float() + o2[1].float()).cpu()
    assert (full - z).abs().mean() < (o2[0].float().cpu() - z).abs().mean()


def test_split_operands_refused_where_unsupported():
    inputs = orc.make_inputs(1, 1, 64, 128, torch.bfloat16, seed=1)
    with pytest.raises(RuntimeError, match="does not support"):
        util.run_tdp(inputs, 0.1, True, backward=False, flags=SPLIT)
    inputs = orc.make_inputs(1, 1, 64, 64, torch.float32, seed=1)
    with pytest.raises(RuntimeError, match="does not support"):
        util.run_tdp(inputs, 0.1, True, backward=False, flags=SPLIT)


def test_mfma_forward_large_values_and_logits():
    """Values in the thousands together with scores spanning hundreds: the fast sweep judges its exponent range
    by the row sums alone (every P is at most its row sum), so the value accumulators must stay finite whenever
    it is accepted, and the repeat sweep must take over where it is not."""
    inputs = orc.make_inputs(1, 2, 160, 64, torch.bfloat16, seed=31)
    inputs[1] = (inputs[1].float() * 5).bfloat16()
    inputs[2] = (inputs[2].float() * 5).bfloat16()
    inputs[3] = (inputs[3].float() * 2048).bfloat16()
    inputs[4] = (inputs[4].float() * 64).bfloat16()
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True)
    for flags in (FORCE_MFMA,):
        out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=flags)
        assert torch.isfinite(out).all()
        scale = z.abs().max()
        err = (out - z).abs() / scale
        assert (err > 2e-2).float().mean() < 0.01 and err.max() < 0.2, (err.max(), (err > 2e-2).float().mean())


@pytest.mark.parametrize("B,H,T,D,seed,windows", [(2, 5, 32, 64, 13, (None,) * 4), (1, 9, 64, 128, 50, (None,) * 4),
                                                  (1, 2, 449, 64, 19, (None,) * 4), (1, 3, 200, 32, 7, (None,) * 4),
                                                  (1, 3, 300, 64, 5, (100, 64, 33, 16))])
def test_fp16_scores_beyond_the_half_precision_range(B, H, T, D, seed, windows):
    """fp16 tensors with Q three times larger: exp2 of a score above 16 is inf in half precision.  The fast
    sweep also runs the virtual rows (q, k > q) of the diagonal k-tile, which no check looks at; what they
    leave in their accumulators (inf, NaN) must not reach the output through a zero weight.  Forward and all
    five gradients against the oracle."""
    print(f"case fp16 range {B, H, T, D} seed {seed} {windows}", flush=True)
    inputs = list(orc.make_inputs(B, H, T, D, torch.float16, seed=seed))
    inputs[0] = (inputs[0].float() * 3).half()
    alpha = 1 / math.sqrt(D)
    z, _, grads = util.oracle_tdp(inputs, alpha, True, windows)
    out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
    assert torch.isfinite(out).all() and all(torch.isfinite(x).all() for x in g)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        # Q three times larger sharpens the softmax: one element in 10^4 may reach 1.5 times the tolerance
        util.assert_mostly_close(name, a, b, **LOWP, outlier_frac=1e-4, outlier_scale=1.5)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shapes_mfma_against_fp32_kernels(seed):
    """Seeded random draws of (B, H, T, D, dtype, causal, windows): the MFMA kernels against the fp32 VALU
    kernels of the same library on the same 16-bit inputs (both go through the C ABI; the fp32 kernels are
    pinned to the oracle by the tests above).  Every third case scales Q by 3: finiteness and agreement there
    too (fp16 scores beyond the half-precision range included)."""
    import random

    rng = random.Random(seed)
    for it in range(12):
        D = rng.choice([32, 64, 128])
        T = rng.choice([1, 7, 31, 32, 33, 63, 64, 65, 95, 127, 129, 191, 200, 257, 320, 449])
        B, H = rng.choice([(1, 1), (1, 3), (2, 5), (1, 9), (3, 3)])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        causal = rng.random() < 0.85
        windows = (None,) * 4
        if rng.random() < 0.7:
            windows = tuple(rng.choice([0, 1, 2, 5, 16, 31, 32, 33, 64, 100, 200, T, 2 * T]) for _ in range(4))
        qscale = 3 if it % 3 == 2 else 1
        print(f"case random {seed}.{it}: {B, H, T, D} {dtype} causal={causal} {windows} q*{qscale}", flush=True)
        inputs = list(orc.make_inputs(B, H, T, D, dtype, seed=100 * seed + it))
        inputs[0] = (inputs[0].float() * qscale).to(dtype)
        alpha = 1 / math.sqrt(D)
        a, ga = util.run_tdp(inputs, alpha, causal, windows, flags=FORCE_MFMA)
        b, gb = util.run_tdp(inputs, alpha, causal, windows, flags=FORCE_GENERIC)
        assert torch.isfinite(a).all() and all(torch.isfinite(x).all() for x in ga)
        # scores three times larger sharpen the softmax: the 16-bit rounding of P and dS then shows in the
        # gradients' cancellations, so those cases get three times the tolerance
        tol = dict(rtol=LOWP["rtol"] * qscale, atol=LOWP["atol"] * qscale)
        # not a parity check (both sides are this library): 0.1 % of the elements may reach 4 times the tolerance
        util.assert_mostly_close("out", a, b, **tol, outlier_frac=1e-3, outlier_scale=4.0)
        for name, x, y in zip(util.NAMES, ga, gb):
            util.assert_mostly_close(name, x, y, **tol, outlier_frac=1e-3, outlier_scale=4.0)


def test_mfma_and_generic_agree_bf16():
    inputs = orc.make_inputs(1, 2, 192, 64, torch.bfloat16, seed=23)
    a, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)
    b, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_GENERIC)
    util.assert_close("out", a, b, **LOWP)


def test_force_mfma_refuses_unsupported():
    inputs = orc.make_inputs(1, 1, 32, 32, torch.float32, seed=24)
    with pytest.raises(RuntimeError, match="does not support"):
        util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)


def test_config3_headline_forward_subset():
    """B=4 H=8 T=1024 D=64 bf16 causal on the GPU; the oracle (chunked dense, CPU) checks all rows
    of three heads."""
    print("case config3 forward", flush=True)
    inputs = orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=3)
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False)
    for (b, h) in ((0, 0), (2, 5), (3, 7)):
        z, lse, _ = orc.tdp_forward_backward_chunked(*(t[b, h].float() for t in inputs), 1 / 8, True,
                                                     q_chunk=64, need_grads=False)
        util.assert_close(f"out[{b},{h}]", out[b, h], z, **LOWP)


@pytest.mark.parametrize("seq_len,row_blocks", [(512, [(0, 512)]), (1024, [(0, 64), (480, 544), (960, 1024)]),
                                                (2048, [(0, 32), (1000, 1032), (2016, 2048)]),
                                                (4096, [(2040, 2056), (4080, 4096)])])
def test_config5_long_sequence_forward(seq_len, row_blocks):
    """B=1 H=16 D=128 bf16 causal, alpha = 1/sqrt(D), T = 512 .. 4096: blocks of query rows of two heads
    against the chunked dense oracle, and device memory beyond the inputs stays O(B H T D): the output,
    the log-sum-exp and one transposed copy of SiLU(V1), never a score plane."""
    print(f"case config5 forward T={seq_len}", flush=True)
    alpha = 1 / math.sqrt(128)
    inputs = orc.make_inputs(1, 16, seq_len, 128, torch.bfloat16, seed=5, n=5)
    dev = [t.cuda() for t in inputs]
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    with torch.no_grad():
        out = flash_trittention(*dev, softmax_scale=alpha, k1_window=None, k2_window=None, kk_left=None,
                                kk_right=None, causal=True)
    torch.cuda.synchronize()
    extra = torch.cuda.max_memory_allocated() - before
    one_tensor = 16 * seq_len * 128 * 2
    assert extra <= 2.5 * one_tensor + (1 << 20), (extra, one_tensor)
    out = out.cpu()
    for h in (3, 15):
        for lo, hi in row_blocks:
            z, _, _ = orc.tdp_forward_backward_chunked(*(t[0, h].float() for t in inputs), None, alpha, True,
                                                       q_chunk=16 if seq_len > 2048 else 64, need_grads=False,
                                                       rows=(lo, hi))
            util.assert_close(f"out[{h}, {lo}:{hi}]", out[0, h, lo:hi].float(), z, **LOWP)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seq_len", [1, 33, 100, 256, 300])
def test_mfma_backward_bf16(seq_len, causal):
    """MFMA forward + backward (FORCE_MFMA), all five gradients, ragged lengths included."""
    print(f"case mfma bwd T={seq_len} causal={causal}", flush=True)
    inputs = orc.make_inputs(1, 3, seq_len, 64, torch.bfloat16, seed=seq_len + 5)
    z, _, grads = util.oracle_tdp(inputs, 1 / 8, causal)
    out, g = util.run_tdp(inputs, 1 / 8, causal, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        if seq_len > 1:  # at T=1 dq, dk1, dk2 are exactly zero in exact arithmetic
            assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seq_len", [1, 33, 100, 256, 300])
@pytest.mark.parametrize("shape", ["w4", "w8", "q16"])
def test_mfma_backward_d128_bf16(seq_len, causal, shape, tune):
    """Head dimension 128, the three shapes of the backward kernel: 32 queries per wave with one wave per SIMD and
    all 128 gradient columns / two waves per SIMD and one half of them, and 16 queries per wave on 16x16x32
    tiles (the default)."""
    print(f"case mfma bwd D=128 T={seq_len} causal={causal} shape={shape}", flush=True)
    tune(_lib.TUNE_BWD128_WAVES, int(shape[1:]))
    inputs = orc.make_inputs(1, 3, seq_len, 128, torch.bfloat16, seed=seq_len + 7)
    alpha = 1 / math.sqrt(128)
    z, _, grads = util.oracle_tdp(inputs, alpha, causal)
    out, g = util.run_tdp(inputs, alpha, causal, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        if seq_len > 1:
            assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("windows", WINDOWS)
@pytest.mark.parametrize("seq_len", [33, 100, 300])
def test_mfma_backward_windows_bf16(seq_len, windows, D):
    """Windowed masks on the MFMA backward (rounds and steps over the band only), all five gradients."""
    print(f"case mfma bwd windows T={seq_len} {windows} D={D}", flush=True)
    inputs = orc.make_inputs(1, 2, seq_len, D, torch.bfloat16, seed=seq_len + D + 3 * sum(windows))
    alpha = 1 / math.sqrt(D)
    z, _, grads = util.oracle_tdp(inputs, alpha, True, windows)
    out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        if b.abs().max() > 0:
            assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("D", [64, 128])
def test_mfma_windows_fp16_batched(D):
    """fp16, several batch entries and heads, odd window sizes: forward and all five gradients."""
    windows = (33, 47, 9, 12)
    inputs = orc.make_inputs(2, 3, 150, D, torch.float16, seed=77 + D)
    alpha = 1 / math.sqrt(D)
    z, _, grads = util.oracle_tdp(inputs, alpha, True, windows)
    out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("splits", [2, 5, 16])
def test_mfma_backward_row_splits(splits, D, tune):
    """The rows of a query tile dealt out to several workgroups (what small grids get): dQ then goes
    through an fp32 accumulator like the row gradients.  Windowed and full masks, ragged length."""
    tune(_lib.TUNE_BWD_SPLITS, splits)
    alpha = 1 / math.sqrt(D)
    for windows in ((None,) * 4, (40, 100, 20, 7)):
        inputs = orc.make_inputs(1, 3, 203, D, torch.bfloat16, seed=splits + D)
        z, _, grads = util.oracle_tdp(inputs, alpha, True, windows)
        out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
        util.assert_close("out", out, z, **LOWP)
        for name, a, b in zip(util.NAMES, g, grads):
            util.assert_mostly_close(name, a, b, **LOWP)
            assert util.rel_err(a, b) <= 5e-2, (name, windows, util.rel_err(a, b))


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_mfma_forward_k_splits(splits, D, tune):
    """The k-tiles of a query tile dealt out to several workgroups and joined by the merge kernel (what
    small grids get): full, non-causal and windowed masks at a ragged length.  Parts with no k-tile at all
    (early query tiles) must drop out of the merge.  The backward reads the merged log-sum-exp."""
    tune(_lib.TUNE_FWD_SPLITS, splits)
    alpha = 1 / math.sqrt(D)
    inputs = orc.make_inputs(1, 3, 203, D, torch.bfloat16, seed=splits + D)
    for causal, windows in ((True, (None,) * 4), (False, (None,) * 4), (True, (40, 100, 20, 7))):
        z, _, grads = util.oracle_tdp(inputs, alpha, causal, windows)
        out, g = util.run_tdp(inputs, alpha, causal, windows, flags=FORCE_MFMA)
        util.assert_close("out", out, z, **LOWP)
        for name, a, b in zip(util.NAMES, g, grads):
            util.assert_mostly_close(name, a, b, **LOWP)


@pytest.mark.parametrize("splits", [1, 4])
def test_mfma_forward_k_splits_large_logits(splits, tune):
    """Scores spanning hundreds with the k-tiles split: every part goes through the repeat sweep with its own
    reference maximum, and the merge must bring them to a common one.  Same statistical bound as the
    unsplit large-logit case; split and unsplit runs must agree far more closely than either does with the
    oracle (they round the same products)."""
    inputs = orc.make_inputs(1, 2, 160, 64, torch.bfloat16, seed=22)
    inputs[1] = (inputs[1].float() * 6).bfloat16()
    inputs[2] = (inputs[2].float() * 6).bfloat16()
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True)
    tune(_lib.TUNE_FWD_SPLITS, 1)
    whole, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)
    tune(_lib.TUNE_FWD_SPLITS, splits)
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False, flags=FORCE_MFMA)
    assert torch.isfinite(out).all()
    err = (out - z).abs()
    assert (err > 5e-2).float().mean() < 0.01 and err.max() < 0.5, (err.max(), (err > 5e-2).float().mean())
    assert (out - whole).abs().max() <= 2e-2, (out - whole).abs().max()


def test_small_grid_forward_splits_by_itself():
    """B=1 H=2 T=256 D=64: 32 query tiles, far below the split threshold, so the launcher splits four ways
    by itself; output and (through the backward, which reads the log-sum-exp) gradients against the oracle,
    and the workspace query covers the parts."""
    from flash_trittention import _lib

    alpha = 1 / 8
    inputs = orc.make_inputs(1, 2, 256, 64, torch.bfloat16, seed=77)
    z, _, grads = util.oracle_tdp(inputs, alpha, True)
    out, g = util.run_tdp(inputs, alpha, True, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
    need = _lib.lib().tritt_tdp_fwd_workspace_bytes(1, 2, 256, 64, _lib.TRITT_BF16, 1, 256, 256, 256, 256, FORCE_MFMA)
    assert need == 2 * 64 * 256 * 2 + 2 * 256 * 4 * 66 * 4, need


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("windows", [(128, 128, 32, 32), (64, 64, 16, 16), (32, 90, 8, 60), (90, 32, 33, 0), (17, 5, 40, 40),
                                     (3, 100, 1, 2)])
def test_band_resident_forward_matches_streaming_and_oracle(windows, D, tune):
    """Narrow windows take the band-resident forward (the whole band of a 32-query tile in LDS); switched off,
    the streaming windowed kernel takes the same problem.  Both against the oracle, and against each other
    far more tightly (they round the same products).  T = 333: eleven query tiles, the last one ragged;
    where the band of a head dimension does not fit in LDS both runs are the streaming kernel."""
    alpha = 1 / math.sqrt(D)
    inputs = orc.make_inputs(1, 2, 333, D, torch.bfloat16, seed=D + windows[0])
    z, _, grads = util.oracle_tdp(inputs, alpha, True, windows)
    out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
    tune(_lib.TUNE_FWD_BAND, -1)
    ref, _ = util.run_tdp(inputs, alpha, True, windows, backward=False, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    util.assert_close("out vs streaming", out, ref, rtol=1e-2, atol=4e-3)
    for name, a, b in zip(util.NAMES, g, grads):  # the backward reads the band kernel's log-sum-exp
        util.assert_mostly_close(name, a, b, **LOWP)


def test_band_resident_forward_large_logits():
    """Scores spanning hundreds under a narrow window: single waves leave the fast sweep and repeat their
    k-tile with the online softmax, and k-tiles with different reference maxima meet in the merge."""
    inputs = orc.make_inputs(1, 2, 160, 64, torch.bfloat16, seed=23)
    inputs[1] = (inputs[1].float() * 6).bfloat16()
    inputs[2] = (inputs[2].float() * 6).bfloat16()
    windows = (70, 50, 20, 30)
    z, _, _ = util.oracle_tdp(inputs, 1 / 8, True, windows)
    out, _ = util.run_tdp(inputs, 1 / 8, True, windows, backward=False, flags=FORCE_MFMA)
    assert torch.isfinite(out).all()
    err = (out - z).abs()
    assert (err > 5e-2).float().mean() < 0.01 and err.max() < 0.5, (err.max(), (err > 5e-2).float().mean())


@pytest.mark.parametrize("T,D,windows", [(8192, 64, (128, 128, 32, 32)), (8192, 128, (64, 64, 32, 32)),
                                         (4096, 64, (300, 300, 64, 64)), (6000, 32, (200, 90, 17, 50))])
def test_long_sequences_under_windows(T, D, windows):
    """Windowed masks are how long sequences become affordable: forward and all five gradients at T = 4096 ..
    8192 (band-resident forward where the band fits in LDS, streaming forward otherwise, banded backward)
    against the oracle evaluated in chunks of query rows over the keys their windows can reach."""
    print(f"case long windows T={T} D={D} {windows}", flush=True)
    alpha = 1 / math.sqrt(D)
    kw = dict(zip(("k1_window", "k2_window", "kk_left", "kk_right"), windows))
    inputs = orc.make_inputs(1, 2, T, D, torch.bfloat16, seed=T % 1000 + D)
    out, g = util.run_tdp(inputs, alpha, True, windows, flags=FORCE_MFMA)
    for h in range(2):
        z, _, grads = orc.tdp_forward_backward_chunked(*(t[0, h].float() for t in inputs), alpha, True, q_chunk=128, **kw)
        util.assert_close(f"out[{h}]", out[0, h], z, **LOWP)
        for name, a, b in zip(util.NAMES, g, grads):
            util.assert_mostly_close(f"{name}[{h}]", a[0, h], b, **LOWP)


@pytest.mark.parametrize("B,H,T,D,windows", [(7, 7500, 640, 64, (None,) * 4), (5, 8000, 512, 128, (64, 64, 32, 32))])
def test_tensors_of_more_than_2_31_elements(B, H, T, D, windows):
    """Element offsets beyond 32 bits (4-5 GB per bf16 tensor, up to ~130 GB of device memory with the
    backward's workspace): the tuned D=64 kernels on full windows, and the band-resident forward and banded
    backward at D=128; the heads around element 2^31 and the last one against the oracle."""
    print(f"case beyond 2^31 elements {B, H, T, D} {windows}", flush=True)
    util.check_offsets_beyond_32_bits("tdp", B, H, T, D, windows)


@pytest.mark.parametrize("shape", [(0, 2, 16, 32), (2, 0, 16, 32), (2, 2, 0, 64)])
def test_empty_inputs_give_empty_results(shape):
    inputs = [torch.zeros(shape, dtype=torch.bfloat16) for _ in range(6)]
    out, grads = util.run_tdp(inputs, 0.125, True, (None,) * 4)
    assert out.shape == shape
    assert all(g.shape == shape for g in grads)
    out, _ = util.run_tdp(inputs, 0.125, True, (4, 4, 2, 2), backward=False)
    assert out.shape == shape


@pytest.mark.parametrize("shape", [(2, 4, 256, 64, (None,) * 4), (1, 3, 200, 128, (None,) * 4), (1, 2, 300, 64, (64, 64, 16, 16))])
def test_forward_and_backward_replay_from_a_hip_graph(shape):
    """The library only launches kernels on the stream it is given (no allocation, copy, memset or
    synchronisation inside), so a forward + backward can be captured into a HIP graph once and replayed for
    launch-bound small problems.  Three replays on fresh inputs, with eager work and synchronisations in between,
    each against the eager result of the same inputs, bit for bit (O and all five gradients)."""
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention

    B, H, T, D, windows = shape
    alpha = 1 / math.sqrt(D)
    kw = dict(softmax_scale=alpha, k1_window=windows[0], k2_window=windows[1], kk_left=windows[2], kk_right=windows[3],
              causal=True)
    static = [t.cuda().requires_grad_(True) for t in orc.make_inputs(B, H, T, D, torch.bfloat16, seed=1)[:5]]
    static_do = torch.zeros(B, H, T, D, dtype=torch.bfloat16, device="cuda")

    def step():
        out = flash_trittention(*static, **kw)
        grads = torch.autograd.grad(out, static, static_do)
        return out, grads

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_grads = step()
    for rep in range(3):
        fresh = orc.make_inputs(B, H, T, D, torch.bfloat16, seed=10 + rep)
        with torch.no_grad():
            for dst, src in zip(static, fresh[:5]):
                dst.copy_(src)
            static_do.copy_(fresh[5])
        graph.replay()
        torch.cuda.synchronize()
        got_out, got_grads = g_out.clone(), [g.clone() for g in g_grads]
        e_out, e_grads = step()   # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got_out, e_out), rep
        for name, a, b in zip(util.NAMES, got_grads, e_grads):
            assert torch.equal(a, b), f"{name} replay {rep}"
        z, _, ref = util.oracle_tdp(fresh, alpha, True, windows)
        util.assert_close("out vs oracle", got_out.float().cpu(), z, **LOWP)


def test_unaligned_views_are_copied():
    """Contiguous views that start in the middle of a storage (2-byte aligned) are accepted: the host side
    copies them to aligned memory before the library sees them."""
    inputs = orc.make_inputs(1, 2, 70, 64, torch.bfloat16, seed=79)
    z, _, grads = util.oracle_tdp(inputs, 1 / 8, True)
    shifted = []
    for t in inputs:
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device="cuda")
        view = buf[1:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 != 0 and view.is_contiguous()
        shifted.append(view)
    out, g = util.run_tdp(shifted, 1 / 8, True, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)


def test_mfma_windows_ignored_without_causal():
    """causal=False ignores the windows (as the naive reference module does)."""
    inputs = orc.make_inputs(1, 2, 100, 64, torch.bfloat16, seed=78)
    a, ga = util.run_tdp(inputs, 1 / 8, False, (5, 3, 4, 1), flags=FORCE_MFMA)
    b, gb = util.run_tdp(inputs, 1 / 8, False, flags=FORCE_MFMA)
    assert torch.equal(a, b)
    for x, y in zip(ga, gb):
        util.assert_close("grad", x, y, **LOWP)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("seq_len", [1, 33, 100, 256, 300])
def test_mfma_backward_d32_bf16(seq_len, causal):
    """Head dimension 32 (row tiles of 64 bytes): forward and all five gradients."""
    print(f"case mfma bwd D=32 T={seq_len} causal={causal}", flush=True)
    inputs = orc.make_inputs(2, 3, seq_len, 32, torch.bfloat16, seed=seq_len + 9)
    alpha = 1 / math.sqrt(32)
    z, _, grads = util.oracle_tdp(inputs, alpha, causal)
    out, g = util.run_tdp(inputs, alpha, causal, flags=FORCE_MFMA)
    util.assert_close("out", out, z, **LOWP)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        if seq_len > 1:
            assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


def test_mfma_backward_d128_fp16_matches_generic():
    """Head dimension 128, fp16, several batch entries and heads: MFMA kernels against the fp32 kernels."""
    inputs = orc.make_inputs(2, 5, 150, 128, torch.float16, seed=33)
    alpha = 1 / math.sqrt(128)
    _, ga = util.run_tdp(inputs, alpha, True, flags=FORCE_MFMA)
    _, gb = util.run_tdp(inputs, alpha, True, flags=FORCE_GENERIC)
    for name, a, b in zip(util.NAMES, ga, gb):
        util.assert_mostly_close(name, a, b, **LOWP)
        assert util.rel_err(a, b) <= 5e-2, (name, util.rel_err(a, b))


def test_mfma_backward_fp16():
    inputs = orc.make_inputs(2, 2, 130, 64, torch.float16, seed=31)
    z, _, grads = util.oracle_tdp(inputs, 1 / 8, True)
    out, g = util.run_tdp(inputs, 1 / 8, True, flags=FORCE_MFMA)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_close(name, a, b, **LOWP)


def test_config3_headline_backward_subset():
    """B=4 H=8 T=1024 D=64 bf16 causal, all five gradients; oracle (chunked dense fp32 on the
    CPU) on two heads, all rows."""
    print("case config3 backward", flush=True)
    inputs = orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=3)
    out, g = util.run_tdp(inputs, 1 / 8, True)
    for (b, h) in ((0, 1), (3, 6)):
        z, lse, grads = orc.tdp_forward_backward_chunked(*(t[b, h].float() for t in inputs), 1 / 8, True,
                                                         q_chunk=64, need_grads=True)
        util.assert_close(f"out[{b},{h}]", out[b, h], z, **LOWP)
        for name, a, ref in zip(util.NAMES, g, grads):
            util.assert_close(f"{name}[{b},{h}]", a[b, h], ref, **LOWP)
            assert util.rel_err(a[b, h], ref) <= 2e-2, (name, util.rel_err(a[b, h], ref))


def test_d128_backward_at_sweep_size_subset():
    """B=1 H=16 T=1024 D=128 bf16 causal (a shape of the sequence-length sweep, with its backward): forward and all
    five gradients of two heads, all rows, against the chunked dense fp32 oracle; the other heads through the
    bitwise head-permutation property."""
    print("case D=128 T=1024 backward", flush=True)
    alpha = 1 / math.sqrt(128)
    inputs = orc.make_inputs(1, 16, 1024, 128, torch.bfloat16, seed=9)
    out, g = util.run_tdp(inputs, alpha, True)
    for h in (2, 13):
        z, lse, grads = orc.tdp_forward_backward_chunked(*(t[0, h].float() for t in inputs), alpha, True, q_chunk=64,
                                                         need_grads=True)
        util.assert_close(f"out[{h}]", out[0, h], z, **LOWP)
        for name, a, ref in zip(util.NAMES, g, grads):
            util.assert_close(f"{name}[{h}]", a[0, h], ref, **LOWP)
            assert util.rel_err(a[0, h], ref) <= 2e-2, (name, util.rel_err(a[0, h], ref))
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(2))
    out2, g2 = util.run_tdp([t[:, perm].contiguous() for t in inputs], alpha, True)
    assert torch.equal(out2, out[:, perm])
    for name, a, b in zip(util.NAMES, g2, g):
        assert torch.equal(a, b[:, perm]), name


# ------------------------------------------------- full-size properties (no oracle: every head is checked)
def _headline_inputs(seed=5):
    return orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=seed)


def test_config3_heads_are_independent_and_order_free():
    """Permuting the (batch, head) slices permutes outputs and all five gradients bit for bit (one owner per
    element, or order-independent fixed-point accumulation)."""
    inputs = _headline_inputs()
    out, g = util.run_tdp(inputs, 1 / 8, True)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(1))
    shuffled = [t.reshape(32, 1024, 64)[perm].reshape(4, 8, 1024, 64).contiguous() for t in inputs]
    out2, g2 = util.run_tdp(shuffled, 1 / 8, True)
    unperm = lambda t: t.reshape(32, 1024, 64)[torch.argsort(perm)].reshape(4, 8, 1024, 64)
    assert torch.equal(unperm(out2), out)
    for name, a, b in zip(util.NAMES, g, g2):
        assert torch.equal(unperm(b), a), name


def test_config3_linear_in_v2_and_do():
    """O is linear in V2; every gradient is linear in dO (same softmax): checked with power-of-two
    factors, which commute with 16-bit rounding, so the forward relation is exact."""
    inputs = _headline_inputs(seed=6)
    out, g = util.run_tdp(inputs, 1 / 8, True)
    scaled = list(inputs)
    scaled[4] = inputs[4] * 4                      # V2 -> 4 V2
    scaled[5] = inputs[5] * 0.5                    # dO -> dO / 2
    out2, g2 = util.run_tdp(scaled, 1 / 8, True)
    assert torch.equal(out2, out * 4)
    # dQ, dK1, dK2, dV1 scale by 4 * 0.5 = 2; dV2 by 0.5
    for name, a, b, f in zip(util.NAMES, g, g2, (2, 2, 2, 2, 0.5)):
        util.assert_close(name, b, a * f, rtol=2e-2, atol=2e-3 * f)


def test_config3_rows_sum_to_one():
    """With V2 = 1 and SiLU(V1) = c (a constant column pattern) the output of every query is c: the
    softmax weights of each of the 4*8*1024 rows sum to one over its (j, k) plane."""
    inputs = _headline_inputs(seed=7)
    c = torch.linspace(-2, 2, 64)
    v1 = torch.empty_like(inputs[3]).copy_(c.expand_as(inputs[3]))
    inputs[3] = v1
    inputs[4] = torch.ones_like(inputs[4])
    out, _ = util.run_tdp(inputs, 1 / 8, True, backward=False)
    want = torch.nn.functional.silu(v1.float()).to(torch.bfloat16).float()
    util.assert_close("out", out, want, rtol=2e-2, atol=2e-2)


# ---------------------------------------------------------------------------------------------------------------
# Range of the backward's common accumulators.  The reference accumulates every gradient in fp32
# (triple_dot_product/kernels/bwd_dk1.py:239-258): no floor under small gradients, non-finite values propagate.
# Here the shares of dK1/dV1/dK2/dV2 (and of a split dQ) are 64-bit fixed point whose scale follows the largest
# |dO| of each (batch, head) slice, so the whole backward is exactly homogeneous in dO for powers of two.

@pytest.mark.parametrize("case", ["config2 bf16 (rows split, dQ accumulated)", "fp32 tensors on the fp32 matrix-core kernels",
                                  "bf16, one workgroup per query tile", "bf16 D=128", "bf16 windowed D=64"])
def test_backward_is_exactly_homogeneous_in_dO(case, tune):
    """dO * 2^-40 (a mean-reduced loss over many tokens, no loss scaling) and dO * 2^+20 (loss scaling) give all
    five gradients bitwise equal to the unscaled run's times that power of two: nothing in the path has an
    absolute resolution or an absolute range."""
    print(f"case homogeneous: {case}", flush=True)
    windows = (None,) * 4
    if case.startswith("config2"):
        inputs, alpha = orc.make_inputs(2, 4, 256, 64, torch.bfloat16, seed=2), 1 / 8
    elif case.startswith("fp32"):
        inputs, alpha = orc.make_inputs(2, 4, 256, 64, torch.float32, seed=3), 1 / 8
    elif case.endswith("per query tile"):
        inputs, alpha = orc.make_inputs(1, 2, 300, 64, torch.bfloat16, seed=4), 1 / 8
        tune(_lib.TUNE_BWD_SPLITS, 1)
    elif case.endswith("D=128"):
        inputs, alpha = orc.make_inputs(1, 3, 203, 128, torch.bfloat16, seed=5), 1 / math.sqrt(128)
    else:
        inputs, alpha, windows = orc.make_inputs(1, 4, 400, 64, torch.bfloat16, seed=6), 1 / 8, (200, 150, 60, 90)
    run = lambda power: util.run_tdp(list(inputs[:5]) + [inputs[5] * 2.0 ** power], alpha, True, windows)[1]
    base = run(0)
    for power in (-40, 20):
        got = run(power)
        for name, a, b in zip(util.NAMES, got, base):
            assert torch.isfinite(a).all(), (name, power)
            assert torch.equal(a, b * 2.0 ** power), (name, power, (a - b * 2.0 ** power).abs().max().item())


@pytest.mark.parametrize("dtype,factor", [(torch.bfloat16, 1e-6), (torch.bfloat16, 1e4), (torch.float32, 4.8e-7),
                                          (torch.float32, 1e4)])
def test_small_and_large_incoming_gradients_against_oracle(dtype, factor):
    """dO of the size `out.mean().backward()` leaves at the headline shape (4.8e-7), and of a scaled loss: every
    gradient meets the usual bar relative to its own magnitude (the tolerances scale with dO)."""
    print(f"case dO x {factor} {dtype}", flush=True)
    inputs = orc.make_inputs(2, 4, 256, 64, dtype, seed=11)
    inputs = list(inputs[:5]) + [(inputs[5].float() * factor).to(dtype)]
    tol = FP32 if dtype == torch.float32 else LOWP
    _, _, grads = util.oracle_tdp(inputs, 1 / 8, True)
    _, g = util.run_tdp(inputs, 1 / 8, True)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a / factor, b / factor, **tol)
        assert util.rel_err(a, b) <= (1e-4 if dtype == torch.float32 else 2e-2), (name, util.rel_err(a, b))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bad", [float("nan"), float("inf")])
def test_non_finite_dO_gives_non_finite_gradients(dtype, bad):
    """A NaN or Inf in dO[b, h, q] reaches dQ[q] and every row j <= q, k <= q of that head's dK1/dV1/dK2/dV2 as
    a non-finite value, as it does through the reference's fp32 accumulators (fp16 training with a GradScaler
    skips the step on exactly that); the other heads keep their gradients bit for bit, and so do the rows of
    the same head past the query tile of q."""
    print(f"case non-finite dO {dtype} {bad}", flush=True)
    B, H, T, D, q = 2, 4, 256, 64, 100
    inputs = orc.make_inputs(B, H, T, D, dtype, seed=13)
    _, base = util.run_tdp(inputs, 1 / 8, True)
    do = inputs[5].clone()
    do[1, 2, q, 5] = bad
    _, g = util.run_tdp(list(inputs[:5]) + [do], 1 / 8, True)
    for name, a, b in zip(util.NAMES, g, base):
        if name == "dq":
            assert not torch.isfinite(a[1, 2, q]).any(), name
        else:
            assert not torch.isfinite(a[1, 2, : q + 1]).any(), name
            assert torch.equal(a[1, 2, 128:], b[1, 2, 128:]), name
        a = a.clone()
        a[1, 2] = b[1, 2]
        assert torch.equal(a, b), f"{name}: another head changed"
