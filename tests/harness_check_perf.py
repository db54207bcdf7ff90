"""Correctness + performance harness that prints parseable CHECK / PERF / RESULT lines, in the format of the
reference's own harness (b200/bench_b200.py:52-157), so numbers can be compared like for like.

    python tests/harness_check_perf.py            (needs a GPU and the built library)

CHECK lines: forward and all five gradients of the HIP path against the CPU oracle on the reference's case grid
(fp32, B=2 H=2 D=32, softmax scale 1/8; T = 64, 100, 33; causal and not; full and (16,16,8,8) windows), with the
reference's tolerances (output rtol 2e-2 / atol 2e-3, gradients atol 5e-3).  PERF lines: forward milliseconds on
the reference's published cases (B=2 H=8 D=64 fp16) beside its published H100 / B200 figures.  Not collected by
pytest (the parity suite proper is tests/test_gpu_*.py); the oracle is used as the checker only.
"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "flash-3-way-attention_amd"))

import torch  # noqa: E402

from flash_trittention.triple_dot_product.flash_trittention import flash_trittention  # noqa: E402
from oracle import trittention_oracle as orc  # noqa: E402
from tests import util  # noqa: E402

SCALE = 1 / 8
# the reference's forward table (h100/README.md:50-53, b200/README.md:53-56): ms of its best kernel per machine
PUBLISHED = [(256, None, "full", 0.298, 0.461), (512, None, "full", 1.451, 2.111), (1024, None, "full", 8.748, 11.61),
             (2048, (128, 128, 32, 32), "win128", 1.163, 1.074)]


def rel_ok(a, b, atol, rtol=2e-2):
    return bool(((a - b).abs() <= atol + rtol * b.abs()).all().item())


def check_correctness():
    ok = True
    for s, causal, kind in [(64, True, "full"), (100, True, "full"), (100, False, "full"), (100, True, "narrow"),
                            (33, True, "full")]:
        windows = (s, s, s, s) if kind == "full" else (16, 16, 8, 8)
        inputs = orc.make_inputs(2, 2, s, 32, torch.float32, seed=s)
        ref, _, ref_grads = util.oracle_tdp(inputs, SCALE, causal, windows)
        out, grads = util.run_tdp(inputs, SCALE, causal, windows)
        fwd_err = (out - ref).abs().max().item()
        errs, grads_pass = {}, True
        for name, a, b in zip(util.NAMES, grads, ref_grads):
            errs[name] = (a - b).abs().max().item()
            grads_pass = grads_pass and rel_ok(a, b, atol=5e-3)
        passed = rel_ok(out, ref, atol=2e-3) and grads_pass
        ok = ok and passed
        print(f"CHECK s={s} causal={causal} win={kind} fwd_err={fwd_err:.2e} "
              + " ".join(f"{k}={v:.2e}" for k, v in errs.items()) + f" -> {'PASS' if passed else 'FAIL'}", flush=True)
    return ok


def bench_forward(iters=30, warmup=5):
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
        print(f"PERF s={s} {label} mi355x_ms={ms:.3f} ref_h100_ms={h100_ms:.3f} ref_b200_ms={b200_ms:.3f} "
              f"speedup={min(h100_ms, b200_ms) / ms:.2f}x", flush=True)


if __name__ == "__main__":
    print(f"gpu={torch.cuda.get_device_name(0)}")
    if not check_correctness():
        print("RESULT correctness=FAIL (skipping perf)")
        sys.exit(1)
    bench_forward()
    print("RESULT correctness=PASS")
