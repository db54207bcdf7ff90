"""Correctness + performance harness that prints parseable CHECK / PERF / RESULT lines, in the format of the
reference's own harness (b200/bench_b200.py:52-157), so numbers can be compared like for like.

    python tests/harness_check_perf.py            (needs a GPU and the built library)

CHECK lines: forward and all five gradients of the HIP path against the CPU oracle on the reference's case grid
(fp32, B=2 H=2 D=32, softmax scale 1/8; T = 64, 100, 33; causal and not; full and (16,16,8,8) windows), with the
reference's tolerances (output rtol 2e-2 / atol 2e-3, gradients atol 5e-3).  The checker is the oracle's drop-in
``Trittention_pytorch`` module, called the way the reference's harness calls the naive module
(b200/bench_b200.py:37-49); the path under test is the package's ``FlashTrittentionModule``.  PERF lines: forward
milliseconds on the reference's published cases (B=2 H=8 D=64 fp16) beside its published H100 / B200 figures.
tests/test_gpu_harness.py runs both legs under pytest; the oracle is used as the checker only.
"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "flash-3-way-attention_amd"))

import torch  # noqa: E402

from flash_trittention import FlashTrittentionModule  # noqa: E402
from flash_trittention.triple_dot_product.flash_trittention import flash_trittention  # noqa: E402
from oracle import trittention_oracle as orc  # noqa: E402
from oracle.triple_dot_product.trittention_pytorch import Trittention_pytorch  # noqa: E402

NAMES = ("dq", "dk1", "dk2", "dv1", "dv2")

SCALE = 1 / 8
# the reference's forward table (h100/README.md:50-53, b200/README.md:53-56): ms of its best kernel per machine
PUBLISHED = [(256, None, "full", 0.298, 0.461), (512, None, "full", 1.451, 2.111), (1024, None, "full", 8.748, 11.61),
             (2048, (128, 128, 32, 32), "win128", 1.163, 1.074)]


def rel_ok(a, b, atol, rtol=2e-2):
    return bool(((a - b).abs() <= atol + rtol * b.abs()).all().item())


def reference(leaves, d_out, causal, windows):
    """Output and gradients of the naive module on the CPU (fp32)."""
    ref = Trittention_pytorch(causal=causal, softmax_scale=SCALE, n_ctx=leaves[0].shape[2], k1_window=windows[0],
                              k2_window=windows[1], kk_left=windows[2], kk_right=windows[3])
    z, *_ = ref(*leaves)
    z.backward(d_out)
    return z.detach(), [t.grad for t in leaves]


def check_correctness(out=print):
    ok = True
    for s, causal, kind in [(64, True, "full"), (100, True, "full"), (100, False, "full"), (100, True, "narrow"),
                            (33, True, "full")]:
        windows = (s, s, s, s) if kind == "full" else (16, 16, 8, 8)
        *inputs, d_out = orc.make_inputs(2, 2, s, 32, torch.float32, seed=s)
        ref, ref_grads = reference([t.clone().requires_grad_(True) for t in inputs], d_out, causal, windows)
        leaves = [t.cuda().requires_grad_(True) for t in inputs]
        module = FlashTrittentionModule(causal=causal, softmax_scale=SCALE, n_ctx=s, k1_window=windows[0],
                                        k2_window=windows[1], kk_left=windows[2], kk_right=windows[3])
        res = module(*leaves)
        res.backward(d_out.cuda())
        res, grads = res.detach().cpu(), [t.grad.cpu() for t in leaves]
        fwd_err = (res - ref).abs().max().item()
        errs, grads_pass = {}, True
        for name, a, b in zip(NAMES, grads, ref_grads):
            errs[name] = (a - b).abs().max().item()
            grads_pass = grads_pass and rel_ok(a, b, atol=5e-3)
        passed = rel_ok(res, ref, atol=2e-3) and grads_pass
        ok = ok and passed
        out(f"CHECK s={s} causal={causal} win={kind} fwd_err={fwd_err:.2e} "
            + " ".join(f"{k}={v:.2e}" for k, v in errs.items()) + f" -> {'PASS' if passed else 'FAIL'}")
    return ok


def bench_forward(iters=30, warmup=5, out=print):
    for s, windows, label, h100_ms, b200_ms in PUBLISHED:
        w = windows or (s, s, s, s)
        q, k1, k2, v1, v2 = (t.cuda() for t in orc.make_inputs(2, 8, s, 64, torch.float16, seed=1, n=5))

        def run():
            with torch.no_grad():
                return flash_trittention(q, k1, k2, v1, v2, softmax_scale=SCALE, k1_window=w[0], k2_window=w[1],
                                         kk_left=w[2], kk_right=w[3], causal=True)

        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / iters
        out(f"PERF s={s} {label} mi355x_ms={ms:.3f} ref_h100_ms={h100_ms:.3f} ref_b200_ms={b200_ms:.3f} "
            f"speedup={min(h100_ms, b200_ms) / ms:.2f}x")


def main(out=print, iters=30):
    out(f"gpu={torch.cuda.get_device_name(0)}")
    if not check_correctness(out):
        out("RESULT correctness=FAIL (skipping perf)")
        return False
    bench_forward(iters=iters, out=out)
    out("RESULT correctness=PASS")
    return True


if __name__ == "__main__":
    sys.exit(0 if main(lambda line: print(line, flush=True)) else 1)
