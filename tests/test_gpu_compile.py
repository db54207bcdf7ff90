"""torch.compile traces the two autograd Functions without graph breaks: under tracing they call the
flash_trittention::* custom ops (torch.library, fake implementations give the output shapes) instead of ctypes.
Backend "aot_eager": the captured forward and backward graphs run eagerly, so no code generator is involved and the
results must equal the eager path's bit for bit."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, H, T, D, dtype, seed):
    from oracle import trittention_oracle as orc

    return [t.cuda() for t in orc.make_inputs(B, H, T, D, dtype, seed=seed)]


@pytest.mark.parametrize("dtype,windows", [(torch.bfloat16, (None,) * 4), (torch.bfloat16, (48, 64, 8, 24)),
                                           (torch.float32, (None,) * 4)])
def test_triple_dot_traces_under_torch_compile(dtype, windows):
    from flash_trittention import flash_trittention

    B, H, T, D = 2, 2, 160, 64
    *ins, d_out = _inputs(B, H, T, D, dtype, seed=21)
    kw = dict(softmax_scale=1 / math.sqrt(D), k1_window=windows[0], k2_window=windows[1], kk_left=windows[2],
              kk_right=windows[3], causal=True)

    def f(q, k1, k2, v1, v2):
        return flash_trittention(q, k1, k2, v1, v2, **kw) * 2.0

    eager = [t.clone().requires_grad_(True) for t in ins]
    f(*eager).backward(d_out)
    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)
    traced = [t.clone().requires_grad_(True) for t in ins]
    out = compiled(*traced)
    out.backward(d_out)
    assert torch.equal(out, f(*eager))
    for a, b in zip(traced, eager):
        assert torch.equal(a.grad, b.grad)


def test_dot_product_sum_traces_under_torch_compile():
    from flash_trittention import TrittentionTriton

    B, H, T, D = 1, 3, 200, 64
    *ins, d_out = _inputs(B, H, T, D, torch.bfloat16, seed=22)
    module = TrittentionTriton(causal=True, softmax_scale=1 / 8, k_diff=50)

    def f(q, k1, k2, v1, v2):
        o, m = module(q, k1, k2, v1, v2)
        return o + 1.0, m

    eager = [t.clone().requires_grad_(True) for t in ins]
    o_e, m_e = f(*eager)
    o_e.backward(d_out)
    compiled = torch.compile(f, backend="aot_eager", fullgraph=True)
    traced = [t.clone().requires_grad_(True) for t in ins]
    o_c, m_c = compiled(*traced)
    o_c.backward(d_out)
    assert torch.equal(o_c, o_e) and torch.equal(m_c, m_e)
    for a, b in zip(traced, eager):
        assert torch.equal(a.grad, b.grad)


def test_custom_ops_pass_opcheck():
    """torch.library.opcheck: schema, fake implementation and functionalisation of the forward ops."""
    from flash_trittention import _ops  # noqa: F401  (registers the ops)

    q, k1, k2, v1, v2, _ = _inputs(1, 2, 96, 64, torch.bfloat16, seed=23)
    torch.library.opcheck(torch.ops.flash_trittention.tdp_fwd.default, (q, k1, k2, v1, v2, 0.125, True, 96, 96, 96, 96, 0),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(torch.ops.flash_trittention.dps_fwd.default, (q, k1, k2, v1, v2, 0.125, True, 96, 0),
                          test_utils=("test_schema", "test_faketensor"))
