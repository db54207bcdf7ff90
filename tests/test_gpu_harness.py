"""The CHECK / PERF / RESULT harness (tests/harness_check_perf.py, the reference's b200/bench_b200.py format) run
under pytest, and the nn.Module front of the triple-dot path against the oracle's drop-in naive module."""
import math
import os
import re

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_check_perf_harness_passes_and_prints_the_reference_format():
    from tests import harness_check_perf as harness

    lines = []

    def out(line):
        lines.append(line)
        print(line, flush=True)

    assert harness.main(out, iters=10)
    checks = [l for l in lines if l.startswith("CHECK ")]
    perfs = [l for l in lines if l.startswith("PERF ")]
    assert len(checks) == 5 and all(l.endswith("-> PASS") for l in checks)
    pat = re.compile(r"^CHECK s=\d+ causal=(True|False) win=(full|narrow) fwd_err=\S+ dq=\S+ dk1=\S+ dk2=\S+ dv1=\S+ "
                     r"dv2=\S+ -> PASS$")
    assert all(pat.match(l) for l in checks), checks
    assert len(perfs) == 4 and all(re.match(r"^PERF s=\d+ \S+ mi355x_ms=\d+\.\d+ ", l) for l in perfs)
    assert lines[-1] == "RESULT correctness=PASS"
    # the harness output of this run is kept as a text file in the run's scratch output folder
    os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
    with open(os.path.join(ROOT, "gpurun_out", "harness_check_perf.txt"), "w") as f:
        f.write("\n".join(lines) + "\n")


@pytest.mark.parametrize("dtype,windows", [(torch.float32, (None,) * 4), (torch.bfloat16, (None,) * 4),
                                           (torch.bfloat16, (40, 64, 8, 24))])
def test_module_matches_the_naive_module(dtype, windows):
    """FlashTrittentionModule against oracle.triple_dot_product.trittention_pytorch.Trittention_pytorch built with
    the same constructor arguments: output and all five gradients."""
    from flash_trittention import FlashTrittentionModule
    from oracle import trittention_oracle as orc
    from oracle.triple_dot_product.trittention_pytorch import Trittention_pytorch

    B, H, T, D = 2, 2, 96, 64
    alpha = 1 / math.sqrt(D)
    kw = dict(causal=True, softmax_scale=alpha, n_ctx=128, k1_window=windows[0], k2_window=windows[1],
              kk_left=windows[2], kk_right=windows[3])
    *inputs, d_out = orc.make_inputs(B, H, T, D, dtype, seed=11)
    ref_leaves = [t.detach().float().clone().requires_grad_(True) for t in inputs]
    z, pre, v_gated, M, L = Trittention_pytorch(**kw)(*ref_leaves)
    z.backward(d_out.float())
    leaves = [t.detach().cuda().requires_grad_(True) for t in inputs]
    module = FlashTrittentionModule(**kw)
    assert not list(module.parameters())
    out = module(*leaves)
    out.backward(d_out.cuda())
    rtol, atol = (1e-4, 2e-5) if dtype == torch.float32 else (5e-2, 2e-2)
    torch.testing.assert_close(out.detach().float().cpu(), z.detach(), rtol=rtol, atol=atol)
    for name, a, b in zip(("dq", "dk1", "dk2", "dv1", "dv2"), leaves, ref_leaves):
        torch.testing.assert_close(a.grad.float().cpu(), b.grad, rtol=rtol, atol=atol, msg=lambda m: f"{name}: {m}")
