"""The oracle (and the independent C brute force) against vectors written by the reference's own
naive modules (tests/golden/make_reference_vectors.py): pins the window-parameter conventions.
The GPU leg checks the HIP path against the same vectors directly."""
import os

import numpy as np
import pytest
import torch

from oracle import brute
from oracle import trittention_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "windowed_masks.npz")
NAMES = ("dq", "dk1", "dk2", "dv1", "dv2")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def _cases(prefix):
    z = np.load(GOLD, allow_pickle=False)
    return sorted(int(k[len(prefix):-4]) for k in z.files if k.startswith(prefix) and k.endswith("_cfg"))


def _inputs(gold, dtype):
    return [torch.from_numpy(gold[n].astype(np.float64)).to(dtype) for n in ("q", "k1", "k2", "v1", "v2", "d_o")]


def _win(v):
    return None if v < 0 else int(v)


@pytest.mark.parametrize("i", _cases("tdp"))
def test_oracle_tdp_matches_reference_vectors(gold, i):
    cfg = gold[f"tdp{i}_cfg"]
    causal, wins = bool(cfg[0]), [_win(v) for v in cfg[1:]]
    ins = _inputs(gold, torch.float64)
    z, _, grads = orc.tdp_forward_backward(*(t[0, 0] for t in ins), float(gold["alpha"]), causal,
                                           k1_window=wins[0], k2_window=wins[1], kk_left=wins[2], kk_right=wins[3])
    np.testing.assert_allclose(z.numpy(), gold[f"tdp{i}_o"][0, 0], rtol=1e-9, atol=1e-11)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"tdp{i}_{n}"][0, 0], rtol=1e-8, atol=1e-10, err_msg=n)


@pytest.mark.parametrize("i", _cases("tdp"))
def test_brute_force_tdp_matches_reference_vectors(gold, i):
    cfg = gold[f"tdp{i}_cfg"]
    T = gold["q"].shape[2]
    causal, wins = bool(cfg[0]), [T if v < 0 else int(v) for v in cfg[1:]]
    ins = [gold[n][0, 0].astype(np.float64) for n in ("q", "k1", "k2", "v1", "v2", "d_o")]
    z, _, *grads = brute.brute(0, *ins, float(gold["alpha"]), causal, wins)
    np.testing.assert_allclose(z, gold[f"tdp{i}_o"][0, 0], rtol=1e-9, atol=1e-11)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g, gold[f"tdp{i}_{n}"][0, 0], rtol=1e-8, atol=1e-10, err_msg=n)


@pytest.mark.parametrize("i", _cases("dps"))
def test_oracle_dps_matches_reference_vectors(gold, i):
    causal, k_diff = bool(gold[f"dps{i}_cfg"][0]), int(gold[f"dps{i}_cfg"][1])
    ins = _inputs(gold, torch.float64)
    z, _, grads = orc.dps_forward_backward(*(t[0, 0] for t in ins), float(gold["alpha"]), causal, k_diff=k_diff)
    np.testing.assert_allclose(z.numpy(), gold[f"dps{i}_o"][0, 0], rtol=1e-9, atol=1e-11)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"dps{i}_{n}"][0, 0], rtol=1e-8, atol=1e-10, err_msg=n)
    ins = [gold[n][0, 0].astype(np.float64) for n in ("q", "k1", "k2", "v1", "v2", "d_o")]
    zb, _, *gb = brute.brute(1, *ins, float(gold["alpha"]), causal, [k_diff])
    np.testing.assert_allclose(zb, gold[f"dps{i}_o"][0, 0], rtol=1e-9, atol=1e-11)
    for n, g in zip(NAMES, gb):
        np.testing.assert_allclose(g, gold[f"dps{i}_{n}"][0, 0], rtol=1e-8, atol=1e-10, err_msg=n)


@pytest.mark.gpu
@pytest.mark.parametrize("i", _cases("tdp"))
def test_hip_tdp_matches_reference_vectors(gold, i):
    from tests.util import run_tdp

    cfg = gold[f"tdp{i}_cfg"]
    causal, wins = bool(cfg[0]), tuple(_win(v) for v in cfg[1:])
    out, grads = run_tdp(_inputs(gold, torch.float32), float(gold["alpha"]), causal, wins)
    np.testing.assert_allclose(out.numpy(), gold[f"tdp{i}_o"], rtol=1e-4, atol=2e-5)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"tdp{i}_{n}"], rtol=1e-4, atol=2e-5, err_msg=n)


@pytest.mark.gpu
@pytest.mark.parametrize("i", _cases("dps"))
def test_hip_dps_matches_reference_vectors(gold, i):
    from tests.util import run_dps

    causal, k_diff = bool(gold[f"dps{i}_cfg"][0]), int(gold[f"dps{i}_cfg"][1])
    out, _, grads = run_dps(_inputs(gold, torch.float32), float(gold["alpha"]), causal, k_diff)
    np.testing.assert_allclose(out.numpy(), gold[f"dps{i}_o"], rtol=1e-4, atol=2e-5)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"dps{i}_{n}"], rtol=1e-4, atol=2e-5, err_msg=n)


def _module_grads(module, ins):
    leaves = [t.clone().requires_grad_(True) for t in ins[:5]]
    res = module(*leaves)
    res[0].backward(ins[5])
    return res, [t.grad for t in leaves]


@pytest.mark.parametrize("i", _cases("tdp"))
def test_naive_module_tdp_returns_match_reference_vectors(gold, i):
    """The drop-in Trittention_pytorch class (triple-dot): all five returns and the autograd gradients."""
    from oracle.triple_dot_product.trittention_pytorch import Trittention_pytorch

    cfg = gold[f"tdp{i}_cfg"]
    wins = [_win(v) for v in cfg[1:]]
    m = Trittention_pytorch(causal=bool(cfg[0]), softmax_scale=float(gold["alpha"]), n_ctx=16, k1_window=wins[0],
                            k2_window=wins[1], kk_left=wins[2], kk_right=wins[3])
    (z, pre, vg, M, L), grads = _module_grads(m, _inputs(gold, torch.float64))
    np.testing.assert_allclose(z.detach().numpy(), gold[f"tdp{i}_o"], rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(pre.detach().numpy(), gold[f"tdp{i}_pre"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(vg.detach().numpy(), gold[f"tdp{i}_vgated"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(M.detach().numpy(), gold[f"tdp{i}_M"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(L.detach().numpy(), gold[f"tdp{i}_L"], rtol=1e-11, atol=1e-12)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"tdp{i}_{n}"], rtol=1e-8, atol=1e-10, err_msg=n)


@pytest.mark.parametrize("i", _cases("dps"))
def test_naive_module_dps_returns_match_reference_vectors(gold, i):
    from oracle.dot_product_sum.trittention_pytorch import Trittention_pytorch

    m = Trittention_pytorch(causal=bool(gold[f"dps{i}_cfg"][0]), softmax_scale=float(gold["alpha"]), n_ctx=16,
                            k_diff=int(gold[f"dps{i}_cfg"][1]))
    (z, pre, vg, M), grads = _module_grads(m, _inputs(gold, torch.float64))
    np.testing.assert_allclose(z.detach().numpy(), gold[f"dps{i}_o"], rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(pre.detach().numpy(), gold[f"dps{i}_pre"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(vg.detach().numpy(), gold[f"dps{i}_vgated"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(M.detach().numpy(), gold[f"dps{i}_M"], rtol=1e-11, atol=1e-12)
    for n, g in zip(NAMES, grads):
        np.testing.assert_allclose(g.numpy(), gold[f"dps{i}_{n}"], rtol=1e-8, atol=1e-10, err_msg=n)
