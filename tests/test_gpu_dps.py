"""GPU parity: dot-product-sum trittention (HIP, through the C ABI) vs the CPU oracle.
Case grid follows the reference's tests/test_dot_product_sum.py:70-142."""
import math

import pytest
import torch

from oracle import trittention_oracle as orc
from tests import util

pytestmark = pytest.mark.gpu

FP32 = dict(rtol=1e-4, atol=2e-5)
LOWP = dict(rtol=5e-2, atol=2e-2)


def check_all(inputs, alpha, causal, k_diff, tol=FP32, rel=1e-4, factorised=False):
    z, lse, grads = util.oracle_dps(inputs, alpha, causal, k_diff, factorised=factorised)
    out, m, g = util.run_dps(inputs, alpha, causal, k_diff)
    util.assert_close("out", out, z, **tol)
    util.assert_close("m", m, lse, rtol=1e-3 if tol is LOWP else 1e-5, atol=2e-2 if tol is LOWP else 1e-4)
    assert util.rel_err(out, z) <= rel
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_close(name, a, b, **tol)
        assert util.rel_err(a, b) <= rel, (name, util.rel_err(a, b))


@pytest.mark.parametrize("seq_len", [33, 64, 100])
@pytest.mark.parametrize("causal", [True, False])
def test_forward_and_backward_fp32(seq_len, causal):
    print(f"case dps fp32 T={seq_len} causal={causal}", flush=True)
    inputs = orc.make_inputs(2, 2, seq_len, 32, torch.float32, seed=seq_len + 1)
    check_all(inputs, 1 / 8, causal, seq_len)


@pytest.mark.parametrize("k_diff", [0, 2, 8])
def test_narrow_k_diff_causal(k_diff):
    print(f"case dps k_diff={k_diff}", flush=True)
    inputs = orc.make_inputs(2, 2, 64, 32, torch.float32, seed=9)
    check_all(inputs, 1 / 8, True, k_diff)


@pytest.mark.parametrize("D", [8, 16, 64, 128])
def test_head_dims_fp32(D):
    inputs = orc.make_inputs(1, 2, 80, D, torch.float32, seed=D + 1)
    check_all(inputs, 1 / math.sqrt(D), True, 80)


def test_large_logits_no_overflow():
    inputs = orc.make_inputs(2, 2, 64, 32, torch.float32, seed=12)
    inputs[1] = inputs[1] * 8.0
    inputs[2] = inputs[2] * 8.0
    z, lse, grads = util.oracle_dps(inputs, 1 / 8, True, 64)
    out, m, g = util.run_dps(inputs, 1 / 8, True, 64)
    assert torch.isfinite(out).all()
    util.assert_close("out", out, z, rtol=1e-3, atol=1e-4)
    for name, a, b in zip(util.NAMES, g, grads):
        assert torch.isfinite(a).all(), name
        util.assert_close(name, a, b, rtol=2e-3, atol=2e-3)


def test_non_contiguous_inputs():
    g = torch.Generator().manual_seed(13)
    q, v1, v2, do = (torch.randn(2, 4, 64, 32, generator=g) for _ in range(4))
    k1 = torch.randn(2, 64, 4, 32, generator=g).transpose(1, 2)
    k2 = torch.randn(2, 64, 4, 32, generator=g).transpose(1, 2)
    inputs = [q, k1, k2, v1, v2, do]
    z, _, grads = util.oracle_dps([t.contiguous() for t in inputs], 1 / 8, True, 64)
    out, m, g_ = util.run_dps(inputs, 1 / 8, True, 64)
    util.assert_close("out", out, z, **FP32)
    for name, a, b in zip(util.NAMES, g_, grads):
        util.assert_close(name, a, b, **FP32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lowp_forward_backward(dtype):
    inputs = orc.make_inputs(2, 2, 256, 64, dtype, seed=14)
    check_all(inputs, 1 / 8, True, 256, tol=LOWP, rel=2e-2)


def test_config4_bf16_T1024():
    """B=4 H=8 T=1024 D=64 bf16 causal.  Oracle: the factorised form (cross-checked against the
    dense cube on the CPU at small T), on a subset of heads to keep the CPU time bounded."""
    inputs = orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=15)
    out, m, g = util.run_dps(inputs, 1 / 8, True, 1024)
    for (b, h) in ((0, 0), (1, 3), (3, 7)):
        sub = [t[b:b + 1, h:h + 1] for t in inputs]
        z, lse, grads = util.oracle_dps(sub, 1 / 8, True, 1024, factorised=True)
        util.assert_close("out", out[b:b + 1, h:h + 1], z, **LOWP)
        util.assert_close("m", m[b:b + 1, h:h + 1], lse, rtol=1e-3, atol=2e-2)
        for name, a, ref in zip(util.NAMES, g, grads):
            util.assert_close(name, a[b:b + 1, h:h + 1], ref, **LOWP)


@pytest.mark.parametrize("seq_len", [1, 33, 100, 257])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_mfma_ragged_lengths(seq_len, causal, D):
    """16-bit tensors take the MFMA kernels (forced, so a silent fall-back would fail)."""
    inputs = orc.make_inputs(1, 2, seq_len, D, torch.bfloat16, seed=20 + seq_len)
    alpha = 1 / math.sqrt(D)
    z, lse, grads = util.oracle_dps(inputs, alpha, causal, seq_len)
    out, m, g = util.run_dps(inputs, alpha, causal, seq_len, flags=2)
    util.assert_close("out", out, z, **LOWP)
    util.assert_close("m", m, lse, rtol=1e-3, atol=2e-2)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)
        if seq_len > 1:
            assert util.rel_err(a, b) <= 3e-2, (name, util.rel_err(a, b))


@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("k_diff", [0, 3, 40, 1000])
def test_mfma_k_diff_band(k_diff, D):
    inputs = orc.make_inputs(2, 2, 150, D, torch.float16, seed=31)
    z, lse, grads = util.oracle_dps(inputs, 1 / 8, True, k_diff)
    out, m, g = util.run_dps(inputs, 1 / 8, True, k_diff, flags=2)
    util.assert_close("out", out, z, **LOWP)
    util.assert_close("m", m, lse, rtol=1e-3, atol=2e-2)
    for name, a, b in zip(util.NAMES, g, grads):
        util.assert_mostly_close(name, a, b, **LOWP)


def test_mfma_matches_generic_kernels():
    inputs = orc.make_inputs(1, 3, 200, 64, torch.bfloat16, seed=32)
    a = util.run_dps(inputs, 1 / 8, True, 50, flags=2)
    b = util.run_dps(inputs, 1 / 8, True, 50, flags=1)
    util.assert_close("out", a[0], b[0], **LOWP)
    util.assert_close("m", a[1], b[1], rtol=1e-3, atol=2e-2)
    for name, x, y in zip(util.NAMES, a[2], b[2]):
        util.assert_mostly_close(name, x, y, **LOWP)


def test_mfma_large_logits():
    """Logits of a few hundred: the online softmax and the chained lse1 bias must not overflow."""
    inputs = [t * (6.0 if i < 3 else 1.0) for i, t in enumerate(orc.make_inputs(1, 2, 128, 64, torch.bfloat16, seed=33))]
    out, m, g = util.run_dps(inputs, 1 / 8, True, 128, flags=2)
    assert torch.isfinite(out).all() and torch.isfinite(m).all()
    assert all(torch.isfinite(x).all() for x in g)
    z, lse, _ = util.oracle_dps(inputs, 1 / 8, True, 128)
    util.assert_close("m", m, lse, rtol=2e-3, atol=5e-2)
    bad = ((out - z).abs() > 5e-2 + 5e-2 * z.abs()).float().mean().item()
    assert bad < 0.01, bad


def test_force_mfma_refused_for_fp32():
    from flash_trittention import _lib

    inputs = orc.make_inputs(1, 1, 32, 64, torch.float32, seed=34)
    with pytest.raises(RuntimeError):
        util.run_dps(inputs, 1 / 8, True, 32, flags=_lib.FLAG_FORCE_MFMA)


def test_head_dim_8_bf16():
    """16-bit tensors with the smallest head dimension: computed by the fp32 kernels, held to the 16-bit bar."""
    inputs = orc.make_inputs(2, 3, 70, 8, torch.bfloat16, seed=8)
    check_all(inputs, 1 / math.sqrt(8), True, 40, tol=LOWP, rel=5e-2)


def test_bitwise_reproducible():
    inputs = orc.make_inputs(1, 2, 200, 64, torch.bfloat16, seed=16)
    a = util.run_dps(inputs, 1 / 8, True, 200)
    b = util.run_dps(inputs, 1 / 8, True, 200)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert torch.equal(x, y)


@pytest.mark.parametrize("T,D,k_diff,causal", [(203, 64, 203, True), (160, 64, 50, True), (96, 128, 1024, True),
                                               (130, 32, 130, True), (64, 64, 64, False), (33, 64, 33, True)])
@pytest.mark.parametrize("waves", [2, 4])
def test_paired_owner_tiles_change_nothing(T, D, k_diff, causal, waves, tune):
    """A workgroup of the MFMA kernels that takes two owner tiles (the long-and-short pairing of full causal
    launches) computes each tile exactly as a workgroup of its own would: forced on and off, every result is
    bitwise the same, odd and even tile counts, banded and unmasked passes included; and it matches the oracle."""
    from flash_trittention import _lib

    print(f"case dps pairing T={T} D={D} k_diff={k_diff} causal={causal} waves={waves}", flush=True)
    inputs = orc.make_inputs(2, 3, T, D, torch.bfloat16, seed=T + D)
    alpha = 1 / math.sqrt(D)
    tune(_lib.TUNE_DPS_WAVES, waves)
    tune(_lib.TUNE_DPS_PAIR, -1)
    a = util.run_dps(inputs, alpha, causal, k_diff, flags=_lib.FLAG_FORCE_MFMA)
    tune(_lib.TUNE_DPS_PAIR, 1)
    b = util.run_dps(inputs, alpha, causal, k_diff, flags=_lib.FLAG_FORCE_MFMA)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    for name, x, y in zip(util.NAMES, a[2], b[2]):
        assert torch.equal(x, y), name
    z, lse, grads = util.oracle_dps(inputs, alpha, causal, k_diff)
    util.assert_close("out", b[0], z, **LOWP)
    for name, x, y in zip(util.NAMES, b[2], grads):
        util.assert_close(name, x, y, **LOWP)


@pytest.mark.parametrize("B,H,T,D,k_diff,causal,dtype", [
    (2, 3, 203, 64, 203, True, torch.bfloat16), (1, 2, 449, 64, 100, True, torch.float16),
    (1, 3, 160, 128, 160, True, torch.bfloat16), (2, 2, 130, 32, 40, True, torch.bfloat16),
    (1, 2, 257, 64, 257, False, torch.bfloat16), (1, 1, 33, 64, 5, True, torch.float16),
    (1, 2, 128, 64, 0, True, torch.bfloat16), (1, 1, 1, 64, 1, True, torch.bfloat16)])
def test_shared_tile_kernels(B, H, T, D, k_diff, causal, dtype, tune):
    """The kernels whose workgroups own 128 rows and read the streamed tiles from an LDS ring (the ones large grids
    take: forward at every head dimension, backward rows and columns at D = 64 and 128), forced on: output, LSE and
    all gradients against the oracle; ragged lengths, bands narrower than a tile, no mask, one row."""
    from flash_trittention import _lib

    print(f"case dps shared-tile kernels B={B} H={H} T={T} D={D} k_diff={k_diff} causal={causal} {dtype}", flush=True)
    inputs = orc.make_inputs(B, H, T, D, dtype, seed=T + D + k_diff)
    alpha = 1 / math.sqrt(D)
    tune(_lib.TUNE_DPS_SHARED, 1)
    out, m, grads = util.run_dps(inputs, alpha, causal, k_diff, flags=_lib.FLAG_FORCE_MFMA)
    tune(_lib.TUNE_DPS_SHARED, -1)
    other = util.run_dps(inputs, alpha, causal, k_diff, flags=_lib.FLAG_FORCE_MFMA)
    z, lse, ref = util.oracle_dps(inputs, alpha, causal, k_diff)
    util.assert_close("out", out, z, **LOWP)
    util.assert_close("m", m, lse, rtol=1e-3, atol=2e-2)
    for name, a, b in zip(util.NAMES, grads, ref):
        util.assert_close(name, a, b, **LOWP)
    # the two forward kernels round the same sums in a different order: a few 16-bit ulps apart
    util.assert_close("out vs the per-tile kernel", out, other[0].float().cpu(), rtol=2e-2, atol=1e-2)


@pytest.mark.parametrize("B,H,fwd_shared", [(16, 16, True), (8, 16, False)])
def test_large_grids_take_the_shared_tile_kernels(B, H, fwd_shared, tune):
    """T=500 D=64: 1024 workgroups of 128 rows (B=16 H=16) send the forward passes and the backward kernels to the
    shared-tile kernels, 512 (B=8 H=16) the backward kernels only.  The default dispatch is bitwise what the knob
    forces for the kernels it picks, and matches the oracle on the heads checked."""
    from flash_trittention import _lib

    T, D = 500, 64
    inputs = orc.make_inputs(B, H, T, D, torch.bfloat16, seed=77)
    default = util.run_dps(inputs, 1 / 8, True, T)
    tune(_lib.TUNE_DPS_SHARED, 1)
    forced = util.run_dps(inputs, 1 / 8, True, T)
    tune(_lib.TUNE_DPS_SHARED, -1)
    never = util.run_dps(inputs, 1 / 8, True, T)
    assert torch.equal(default[0], (forced if fwd_shared else never)[0])
    assert torch.equal(default[1], (forced if fwd_shared else never)[1])
    assert not torch.equal(forced[0], never[0])
    if fwd_shared:  # every kernel of the default path is the forced one
        for name, a, b in zip(util.NAMES, default[2], forced[2]):
            assert torch.equal(a, b), name
    assert not all(torch.equal(a, b) for a, b in zip(default[2], never[2]))
    for b, h in ((0, 0), (B // 2, 9), (B - 1, H - 1)):
        z, lse, grads = util.oracle_dps([t[b:b + 1, h:h + 1] for t in inputs], 1 / 8, True, T)
        util.assert_close("out", default[0][b:b + 1, h:h + 1], z, **LOWP)
        util.assert_close("m", default[1][b:b + 1, h:h + 1], lse, rtol=1e-3, atol=2e-2)
        for name, a, ref in zip(util.NAMES, default[2], grads):
            util.assert_close(name, a[b:b + 1, h:h + 1], ref, **LOWP)


def test_rejects_mismatched_shapes():
    from flash_trittention import TrittentionTriton

    q, k1, k2, v1, v2, _ = (t.cuda() for t in orc.make_inputs(2, 2, 32, 32))
    with pytest.raises(ValueError):
        TrittentionTriton()(q, k1, k2, v1, v2[:, :, :16, :].contiguous())


@pytest.mark.parametrize("seed", [0, 1])
def test_random_shapes_mfma_against_fp32_kernels(seed):
    """Seeded random draws of (B, H, T, D, dtype, causal, k_diff): the MFMA kernels against the fp32 kernels
    of the same library on the same 16-bit inputs; every third case scales Q by 3."""
    import random

    rng = random.Random(seed)
    for it in range(12):
        D = rng.choice([32, 64, 128])
        T = rng.choice([1, 7, 31, 32, 33, 63, 64, 65, 127, 129, 200, 257, 449, 513, 1000])
        B, H = rng.choice([(1, 1), (1, 3), (2, 5), (1, 9), (3, 3)])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        causal = rng.random() < 0.85
        k_diff = rng.choice([0, 1, 2, 5, 31, 32, 33, 100, T, 2 * T, None])
        qscale = 3 if it % 3 == 2 else 1
        print(f"case random {seed}.{it}: {B, H, T, D} {dtype} causal={causal} k_diff={k_diff} q*{qscale}", flush=True)
        inputs = list(orc.make_inputs(B, H, T, D, dtype, seed=100 * seed + it))
        inputs[0] = (inputs[0].float() * qscale).to(dtype)
        alpha = 1 / math.sqrt(D)
        a, ma, ga = util.run_dps(inputs, alpha, causal, k_diff, flags=2)
        b, mb, gb = util.run_dps(inputs, alpha, causal, k_diff, flags=1)
        assert torch.isfinite(a).all() and torch.isfinite(ma).all() and all(torch.isfinite(x).all() for x in ga)
        tol = dict(rtol=5e-2 * qscale, atol=2e-2 * qscale)
        # not a parity check (both sides are this library): 0.1 % of the elements may reach 4 times the tolerance
        loose = dict(outlier_frac=1e-3, outlier_scale=4.0)
        util.assert_mostly_close("out", a, b, **tol, **loose)
        util.assert_mostly_close("m", ma, mb, **tol, **loose)
        for name, x, y in zip(util.NAMES, ga, gb):
            util.assert_mostly_close(name, x, y, **tol, **loose)


def test_tensors_of_more_than_2_31_elements():
    """Element offsets beyond 32 bits: B*H = 52500 heads of T=640, D=64 (4.3 GB per bf16 tensor)."""
    print("case beyond 2^31 elements (7, 7500, 640, 64)", flush=True)
    util.check_offsets_beyond_32_bits("dps", 7, 7500, 640, 64)


@pytest.mark.parametrize("shape", [(0, 2, 16, 32), (2, 0, 16, 32), (2, 2, 0, 32)])
def test_empty_inputs_give_empty_results(shape):
    inputs = [torch.zeros(shape, dtype=torch.bfloat16) for _ in range(6)]
    out, m, grads = util.run_dps(inputs, 0.125, True, 16)
    assert out.shape == shape and m.shape == shape[:3]
    assert all(g.shape == shape for g in grads)


# ------------------------------------------------- full-size properties (config 4: B=4 H=8 T=1024 D=64 bf16)
def test_config4_heads_are_independent_bitwise():
    """Every output element has one owner (no atomics): permuting the (batch, head) slices permutes
    the output, the LSE and all five gradients bit for bit."""
    inputs = orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=41)
    out, m, g = util.run_dps(inputs, 1 / 8, True, 1024)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(2))
    shuffled = [t.reshape(32, 1024, 64)[perm].reshape(4, 8, 1024, 64).contiguous() for t in inputs]
    out2, m2, g2 = util.run_dps(shuffled, 1 / 8, True, 1024)
    inv = torch.argsort(perm)
    unperm = lambda t: t.reshape(32, 1024, -1)[inv].reshape(t.shape)
    assert torch.equal(unperm(out2), out)
    assert torch.equal(unperm(m2.reshape(4, 8, 1024, 1)).reshape(4, 8, 1024), m)
    for a, b in zip(g, g2):
        assert torch.equal(unperm(b), a)


def test_config4_linear_in_v2_and_do():
    """O is linear in V2 and the gradients in dO; power-of-two factors commute with the 16-bit rounding
    of every intermediate, so the relations are exact."""
    inputs = orc.make_inputs(4, 8, 1024, 64, torch.bfloat16, seed=42)
    out, m, g = util.run_dps(inputs, 1 / 8, True, 1024)
    scaled = list(inputs)
    scaled[4] = inputs[4] * 4
    scaled[5] = inputs[5] * 0.5
    out2, m2, g2 = util.run_dps(scaled, 1 / 8, True, 1024)
    assert torch.equal(out2, out * 4)
    assert torch.equal(m2, m)
    for name, a, b, f in zip(util.NAMES, g, g2, (2, 2, 2, 2, 0.5)):
        util.assert_close(name, b, a * f, rtol=1e-2, atol=1e-3 * f)


@pytest.mark.parametrize("shape", [(2, 3, 256, 64, 256), (1, 2, 200, 128, 40)])
def test_forward_and_backward_replay_from_a_hip_graph(shape):
    """A dot-product-sum call is kernel launches only: forward + backward captured into a HIP graph once, three
    replays on fresh inputs with eager work and synchronisations in between, each bitwise equal to the eager
    result of the same inputs (every output element of this path has one owner)."""
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTriton

    B, H, T, D, k_diff = shape
    mod = TrittentionTriton(causal=True, softmax_scale=1 / math.sqrt(D), k_diff=k_diff)
    static = [t.cuda().requires_grad_(True) for t in orc.make_inputs(B, H, T, D, torch.bfloat16, seed=2)[:5]]
    static_do = torch.zeros(B, H, T, D, dtype=torch.bfloat16, device="cuda")

    def step():
        out, m = mod(*static)
        return out, m, torch.autograd.grad(out, static, static_do)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_m, g_grads = step()
    for rep in range(3):
        fresh = orc.make_inputs(B, H, T, D, torch.bfloat16, seed=20 + rep)
        with torch.no_grad():
            for dst, src in zip(static, fresh[:5]):
                dst.copy_(src)
            static_do.copy_(fresh[5])
        graph.replay()
        torch.cuda.synchronize()
        got = [g_out.clone(), g_m.clone()] + [g.clone() for g in g_grads]
        e_out, e_m, e_grads = step()
        torch.cuda.synchronize()
        for a, b in zip(got, [e_out, e_m] + list(e_grads)):
            assert torch.equal(a, b), rep
        z, lse, _ = util.oracle_dps(fresh, 1 / math.sqrt(D), True, k_diff, factorised=True)
        util.assert_close("out vs oracle", got[0].float().cpu(), z, **LOWP)


@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("causal,k_diff", [(True, 250), (True, 37), (True, 0), (False, 250)])
def test_fp32_tensors_on_the_matrix_cores(D, causal, k_diff, tune):
    """fp32 tensors run the three attention kernels on the fp32 MFMA (ragged length, two owner tiles per head and
    more): forward, m and all five gradients at the fp32 bar against the oracle, and against the fp32 VALU
    kernels of the same library (what the reference's fp32 test grid covers: tests/test_dot_product_sum.py:70-118)."""
    from flash_trittention import _lib

    print(f"case dps fp32 mfma D={D} causal={causal} k_diff={k_diff}", flush=True)
    inputs = orc.make_inputs(2, 3, 250, D, torch.float32, seed=D + k_diff)
    alpha = 1 / math.sqrt(D)
    check_all(inputs, alpha, causal, k_diff, factorised=False)
    out, m, g = util.run_dps(inputs, alpha, causal, k_diff)
    tune(_lib.TUNE_F32_VALU, 1)
    out_v, m_v, g_v = util.run_dps(inputs, alpha, causal, k_diff)
    assert not torch.equal(out, out_v), "both runs took the same kernels"
    util.assert_close("out vs VALU kernels", out, out_v, **FP32)
    util.assert_close("m vs VALU kernels", m, m_v, rtol=1e-5, atol=1e-4)
    for name, a, b in zip(util.NAMES, g, g_v):
        util.assert_close(f"{name} vs VALU kernels", a, b, **FP32)


def test_large_logits_with_convert_to_float32_hold_the_16_bit_bar():
    """convert_to_float32=True on 16-bit tensors: fp32 operands throughout (the fp32 matrix-core kernels), as the
    reference's flag asks of its kernels (dot_product_sum/trittention_triton.py:92-119).  Logits of a few hundred,
    where the 16-bit MFMA path is held to a statistical bound, meet the 16-bit tolerance element by element."""
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTriton

    inputs = [t * (6.0 if i < 3 else 1.0) for i, t in enumerate(orc.make_inputs(1, 2, 128, 64, torch.bfloat16, seed=33))]
    z, lse, grads = util.oracle_dps(inputs, 1 / 8, True, 128)
    leaves = [t.cuda().requires_grad_(True) for t in inputs[:5]]
    out, m = TrittentionTriton(causal=True, softmax_scale=1 / 8, k_diff=128, convert_to_float32=True)(*leaves)
    out.backward(inputs[5].cuda())
    util.assert_mostly_close("out", out.detach().float().cpu(), z, **LOWP)
    util.assert_close("m", m.cpu(), lse, rtol=1e-4, atol=1e-3)
    for name, leaf, want in zip(util.NAMES, leaves, grads):
        util.assert_mostly_close(name, leaf.grad.float().cpu(), want, **LOWP)
