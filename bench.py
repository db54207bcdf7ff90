#!/usr/bin/env python3
"""Benchmark of the trittention hot path on one MI355X.

A step = one triple-dot-product forward + backward over one synthetic batch at
B=4 H=8 T=1024 D=64 bf16 causal (inputs resident in HBM before the timed
region).  Prints ONE JSON line.  `value` is the algorithmic TFLOP/s of the
whole step: 16*D*N / time with N = B*H*T(T+1)(2T+1)/6 valid (q,j,k) triples
(forward 4*D*N, backward 12*D*N).  `roofline` covers the dominant kernel (the backward rows
kernel, launched twice per step), `roofline_fwd` the forward kernel; both divide by the
MI355X dense bf16 MFMA peak.
`cpu_baseline` times the CPU oracle (the reference's naive dense formulation)
on a bounded sample on this box's host cores.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-3-way-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3   # dense fp32 MFMA
PEAK_HBM_GBS = 8000.0
NOMINAL_CLOCK_MHZ = 2400.0  # the clock behind the published peak
# HBM bytes per launch, NOT measured live: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script at the
# default workload only, scaled by a plain 256 MiB copy (summary and commands:
# profiles/tdp_fwd_bwd_B4_H8_T1024_D64_bf16_counters.txt).  Reported only when the workload is the default one.
TRAFFIC_SOURCE = "profiles/tdp_fwd_bwd_B4_H8_T1024_D64_bf16_counters.txt (rocprofv3 --pmc, default workload only)"
# 27.4 MiB fetched + 15.0 MiB written: the algorithmic 20 + 4 MiB, and 28 bytes per lane that the kernel's prologue
# spills (a million lanes: ~11 MiB written once; spill-free builds of the kernel measured 2 % slower)
TRAFFIC_FWD = 44.4e6
# average of the two launches: 587 / 527 MiB written (64-bit atomics; the first launch also spills 16-20 bytes per lane), 36 / 39 MiB fetched (some runs: up to 440 MiB in the first
# launch, when its accumulators fall out of their XCD's L2; the bytes are L2 <-> fabric traffic, which the 256 MB Infinity
# Cache absorbs)
TRAFFIC_BWD_ROWS = 624e6


def triples(B, H, T, causal=True):
    return B * H * (T * (T + 1) * (2 * T + 1) // 6 if causal else T ** 3)


def windowed_triples(T, w1, w2, kl, kr):
    """Valid (q, j, k) of one head under the windowed causal mask, by the predicate the kernels use:
    j, k <= q, q - j <= w1, q - k <= w2, k - j <= kl, j - k <= kr."""
    import numpy as np

    total = 0
    for q in range(T):
        j = np.arange(max(0, q - w1), q + 1)
        lo = np.maximum(max(0, q - w2), j - kr)
        hi = np.minimum(q, j + kl)
        total += int(np.maximum(hi - lo + 1, 0).sum())
    return total


def make_inputs(B, H, T, D, dtype, seed=0, n=6):
    """Seeded synthetic inputs: N(0,1) draws from a CPU generator in the order Q, K1, K2, V1, V2, dO, drawn in
    fp32 and then cast (the same draws the parity tests use)."""
    import torch

    g = torch.Generator(device="cpu").manual_seed(seed)
    return [torch.randn(B, H, T, D, generator=g, dtype=torch.float32).to(dtype) for _ in range(n)]


def nominal_clock_mhz():
    """The device's nominal shader clock (hipDeviceAttributeClockRate = 5, kHz) from the HIP runtime the
    process already has loaded; None if the runtime cannot be reached."""
    import ctypes

    for name in ("libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6"):
        try:
            hip = ctypes.CDLL(name)
            v = ctypes.c_int(0)
            if hip.hipDeviceGetAttribute(ctypes.byref(v), 5, 0) == 0 and v.value > 0:
                return v.value / 1e3
        except OSError:
            continue
    return None


def time_events(fn, iters, warmup, torch):
    """Average milliseconds per call, HIP events on the stream the kernels run on
    (torch's current stream, which is the stream handed to the library)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_info():
    """Model string of the host CPU and how many of its cores this process may use."""
    model = None
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    quota = None
    try:
        with open("/sys/fs/cgroup/cpu.max") as f:
            lim, period = f.read().split()
            if lim != "max":
                quota = float(lim) / float(period)
    except (OSError, ValueError):
        pass
    return {"model": model, "os_cpu_count": os.cpu_count(), "affinity": len(os.sched_getaffinity(0)),
            "cgroup_cpu_quota": quota, "OMP_NUM_THREADS": os.environ.get("OMP_NUM_THREADS")}


def mfma_probe(torch, _lib, blocks=2048, iters=4096):
    """Rate of a kernel that does nothing but bf16 MFMAs (tritt_probe_mfma), and the clock it implies."""
    out = torch.empty(blocks * 512, dtype=torch.float32, device="cuda")
    lib = _lib.lib()

    def run():
        _lib.check(lib.tritt_probe_mfma(_lib.ptr(out), blocks, iters, _lib.stream_ptr(out.device)), "tritt_probe_mfma")

    ms = time_events(run, 5, 2, torch)
    tflops = blocks * 8 * iters * 4 * 32768 / ms / 1e9
    return {"tflops": tflops, "ms": ms,
            "implied_clock_mhz": tflops / PEAK_BF16_TFLOPS * NOMINAL_CLOCK_MHZ,
            "what": "a kernel of independent 32x32x16 bf16 MFMAs only, 16 waves per CU: the matrix rate this chip "
                    "sustains; implied clock = rate / 2500 TFLOP/s x 2400 MHz"}


def cpu_baseline(T, D, alpha, seconds_budget=30.0):
    """The oracle's naive dense path (einsum -> mask -> softmax over the flattened (j,k)
    plane -> einsum, gradients by autograd), fp32, on this host's cores: a few heads of the
    headline workload, all T query rows, evaluated in chunks of query rows so the
    [q, j, k] slab stays bounded.  Throughput is algorithmic flops / time."""
    import torch

    from oracle import trittention_oracle as orc

    # every core this process may use: the smaller of its affinity mask, its cgroup quota and an OMP_NUM_THREADS the
    # box sets for its share of the host (oversubscribing a share only slows the ATen kernels down)
    info = cpu_info()
    cores = info["affinity"]
    if info["cgroup_cpu_quota"]:
        cores = min(cores, max(1, int(info["cgroup_cpu_quota"])))
    if info["OMP_NUM_THREADS"] and info["OMP_NUM_THREADS"].isdigit():
        cores = min(cores, int(info["OMP_NUM_THREADS"]))
    torch.set_num_threads(cores)
    max_heads = 8
    full = orc.make_inputs(1, max_heads, T, D, torch.bfloat16, seed=0)
    heads, t0 = 0, time.perf_counter()
    while heads < max_heads:
        ins = [t[0, heads].float() for t in full]
        orc.tdp_forward_backward_chunked(*ins, alpha, True, q_chunk=64, need_grads=True)
        heads += 1
        if time.perf_counter() - t0 >= min(12.0, seconds_budget):
            break
    dt = time.perf_counter() - t0
    flops = 16 * D * triples(1, heads, T)
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "cpu": info,
        "seconds": dt,
        "sample": f"{heads} of the 32 heads of the workload (T={T}, D={D}), all query rows, fwd+bwd, "
                  "dense fp32 in 64-row query chunks, heads one after another until 12 s have passed; "
                  "throughput = algorithmic flops of those heads / time",
    }


def sweep_rows(torch, flash_trittention, dev, steps):
    """BASELINE config 5: triple-dot forward, B=1 H=16 D=128 bf16 causal, T = 512 .. 4096."""
    rows = []
    for Ts in (512, 1024, 2048, 4096):
        ins = [t.to(dev) for t in make_inputs(1, 16, Ts, 128, torch.bfloat16, seed=0, n=5)]
        torch.cuda.reset_peak_memory_stats()
        base_mem = torch.cuda.memory_allocated()

        def f():
            with torch.no_grad():
                return flash_trittention(*ins, softmax_scale=1 / math.sqrt(128), k1_window=None, k2_window=None,
                                         kk_left=None, kk_right=None, causal=True)

        ms = time_events(f, max(3, min(4 * steps, 65536 // Ts)), 3 if Ts <= 2048 else 1, torch)
        fl = 4 * 128 * triples(1, 16, Ts)
        rows.append({"T": Ts, "ms": ms, "tflops": fl / ms / 1e9, "frac_of_bf16_peak": fl / ms / 1e9 / PEAK_BF16_TFLOPS,
                     "extra_device_bytes": torch.cuda.max_memory_allocated() - base_mem,
                     "one_tensor_bytes": 16 * Ts * 128 * 2})
    return rows


def dps_times(torch, dev, B, H, T, D, steps, warmup, dtype=None, k_diff=None):
    """Dot-product-sum forward and backward (events around the Python calls): BASELINE config 4 by default; `dtype`
    and `k_diff` for the reference's own large configurations (scripts/benchmark_dot_product_sum.py:400-510)."""
    from flash_trittention.dot_product_sum.trittention_triton import TrittentionTriton

    dtype = dtype or torch.bfloat16
    k_diff = T if k_diff is None else min(k_diff, T)
    alpha = 1 / math.sqrt(D)
    ins = [t.to(dev) for t in make_inputs(B, H, T, D, dtype, seed=0)]
    lv = [t.clone().requires_grad_(True) for t in ins[:5]]
    mod = TrittentionTriton(causal=True, softmax_scale=alpha, k_diff=k_diff)
    hold = {}

    def f():
        hold["o"] = mod(*lv)[0]

    def b():
        # the gradients are returned, not added into .grad: an accumulation into gradients that earlier iterations
        # left behind (five extra elementwise kernels) is the timing loop's doing, not the operator's
        hold["g"] = torch.autograd.grad(hold["o"], lv, ins[5], retain_graph=True)

    ms_f = time_events(f, steps, max(warmup, 3), torch)
    ms_b = time_events(b, steps, max(warmup, 3), torch)  # the first backward pays one-time set-up
    # the same backward called as an operator, without the autograd engine: at the small shapes the engine's hand-over
    # to its device thread takes longer on the host than the five kernels take on the GPU, and the events above then
    # time the host
    from flash_trittention import _ops
    with torch.no_grad():
        o_op, lse_op = _ops.dps_fwd_impl(*ins[:5], alpha, True, k_diff, 0)
        ms_f_op = time_events(lambda: _ops.dps_fwd_impl(*ins[:5], alpha, True, k_diff, 0), steps, max(warmup, 3), torch)
        ms_b_op = time_events(lambda: _ops.dps_bwd_impl(*ins[:5], o_op, lse_op, ins[5], alpha, True, k_diff, 0), steps,
                              max(warmup, 3), torch)
    n3 = B * H * T * (T + 1) * (T + 2) // 6   # valid (q,s,t) triples of the reference's formulation, k_diff = T
    # (row, column) pairs of the factorised form: the inner attention (t, s) with t - s <= k_diff, the outer (q, t)
    n_in = B * H * sum(min(t + 1, k_diff + 1) for t in range(T))
    n_out = B * H * T * (T + 1) // 2
    elem = 4 if dtype == torch.float32 else 2
    peak = PEAK_F32_TFLOPS if dtype == torch.float32 else PEAK_BF16_TFLOPS
    bytes_f, bytes_b = 6 * B * H * T * D * elem + 4 * B * H * T, 12 * B * H * T * D * elem + 8 * B * H * T
    tf_f, tf_b = 4 * D * (n_in + n_out) / ms_f / 1e9, 10 * D * (n_in + n_out) / ms_b / 1e9
    row = {"fwd_ms": ms_f, "bwd_ms": ms_b, "fwd_ms_operator_call": ms_f_op, "bwd_ms_operator_call": ms_b_op,
           "executed_fwd_tflops": tf_f, "executed_bwd_tflops": tf_b,
           "mfma_frac_fwd": tf_f / peak, "mfma_frac_bwd": tf_b / peak,
           "algorithmic_bytes_fwd": bytes_f, "algorithmic_bytes_bwd": bytes_b,
           "io_gbs_fwd": bytes_f / ms_f / 1e6, "io_gbs_bwd": bytes_b / ms_b / 1e6,
           # the factorised path is bound by HBM (8.6 / 21.5 GFLOP on 25 / 50 MB): fraction of the 8 TB/s floor
           "roofline_fwd": {"bound": "hbm", "achieved": bytes_f / ms_f / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": bytes_f / ms_f / 1e6 / PEAK_HBM_GBS},
           "roofline_bwd": {"bound": "hbm", "achieved": bytes_b / ms_b / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": bytes_b / ms_b / 1e6 / PEAK_HBM_GBS},
           "config": {"workload": f"dot-product-sum fwd+bwd B={B} H={H} T={T} D={D} {str(dtype).split('.')[-1]} causal "
                                  f"k_diff={k_diff}"}}
    if k_diff >= T:
        row["reference_formulation_fwd_tflops_equiv"] = 4 * D * n3 / ms_f / 1e9
    return row


def tdp_times(torch, flash_trittention, dev, B, H, T, D, dtype, steps, warmup, backward=True, convert=False):
    """Triple-dot forward (and backward) milliseconds at one shape, full windows.  `convert`: the reference's
    convert_to_float32=True (what its own benchmark scripts pass: scripts/benchmark_triple_dot_product.py:172)."""
    alpha = 1 / math.sqrt(D)
    q, k1, k2, v1, v2, do = (t.to(dev) for t in make_inputs(B, H, T, D, dtype, seed=0))
    leaves = [t.clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    kw = dict(softmax_scale=alpha, k1_window=None, k2_window=None, kk_left=None, kk_right=None, causal=True,
              convert_to_float32=convert)
    hold = {}

    def fwd():
        with torch.no_grad():
            return flash_trittention(q, k1, k2, v1, v2, **kw)

    def bwd():
        hold["g"] = torch.autograd.grad(hold["o"], leaves, do, retain_graph=True)  # returned, not added into .grad

    n = triples(B, H, T)
    row = {"workload": f"triple-dot B={B} H={H} T={T} D={D} {str(dtype).split('.')[-1]} causal"
                       + (" convert_to_float32=True" if convert else ""),
           "fwd_ms": time_events(fwd, steps, warmup, torch)}
    row["fwd_tflops"] = 4 * D * n / row["fwd_ms"] / 1e9
    if backward:
        hold["o"] = flash_trittention(*leaves, **kw)
        row["bwd_ms"] = time_events(bwd, steps, warmup, torch)
        row["bwd_tflops"] = 12 * D * n / row["bwd_ms"] / 1e9
    return row


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--brief", action="store_true", help="default mode: skip the other BASELINE configurations")
    ap.add_argument("--mode", choices=["both", "fwd", "copy", "sweep", "seqlen", "dps", "dpsrange", "tdp", "published"], default="both",
                    help="fwd: time only the forward (for profiling runs); copy: a plain 256 MiB device copy, "
                         "the known-size kernel the FETCH_SIZE / WRITE_SIZE counters are calibrated against; "
                         "sweep: triple-dot forward at B=1 H=16 D=128 bf16 over T in 512..4096; "
                         "seqlen: the reference's windowed sequence-length sweep (scripts/benchmark_seq_len_range.py:"
                         "11-31,177: B=2 H=2 D=64, k1_window 24, k2_window 22, T = 256..2048 step 256, forward and "
                         "backward, convert_to_float32=True), fp32 tensors as there and bf16; "
                         "dps: dot-product-sum forward+backward at --B --H --T --D; "
                         "dpsrange: the large configurations of the reference's dot-product-sum benchmark "
                         "(scripts/benchmark_dot_product_sum.py:400-510: B=1 H=8 D=64, T = 1024..8192, k_diff 128 / 1024 / "
                         "2048, fp32 and bf16); "
                         "tdp: triple-dot forward+backward at --B --H --T --D with --windows (secondary shapes: "
                         "D=128, windowed masks); "
                         "published: the forward cases the reference publishes timings for (B=2 H=8 D=64 fp16 causal: "
                         "T=256/512/1024 full windows, T=2048 windows 128,128,32,32), its best H100 / B200 figures beside ours")
    ap.add_argument("--windows", default="", help="k1_window,k2_window,kk_left,kk_right for --mode tdp (empty: full)")
    ap.add_argument("--dtype", choices=["bf16", "fp16", "fp32"], default="bf16", help="tensor type for --mode tdp and --mode dps")
    ap.add_argument("--convert", action="store_true", help="--mode tdp: pass convert_to_float32=True")
    ap.add_argument("--B", type=int, default=4)
    ap.add_argument("--H", type=int, default=8)
    ap.add_argument("--T", type=int, default=1024)
    ap.add_argument("--D", type=int, default=64)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every (batch, head) slice is independent, so more GPUs "
                 "only replicate this number; run with --gpus 1")

    import torch

    from flash_trittention import _lib
    from flash_trittention.triple_dot_product.flash_trittention import flash_trittention
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    _lib.lib()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    if args.mode == "copy":
        nbytes = 256 << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        ms = time_events(lambda: dst.copy_(src), args.steps, args.warmup, torch)
        print(json.dumps({"metric": "device copy", "bytes_read": nbytes, "bytes_written": nbytes,
                          "ms_per_step": ms, "value": 2 * nbytes / ms / 1e6, "unit": "GB/s"}), flush=True)
        return
    B, H, T, D = args.B, args.H, args.T, args.D
    alpha = 1 / math.sqrt(D)
    if args.mode == "sweep":
        rows = sweep_rows(torch, flash_trittention, dev, args.steps)
        print(json.dumps({"metric": "triple-dot trittention fwd TFLOP/s vs T", "unit": "TFLOP/s",
                          "config": {"workload": "triple-dot fwd B=1 H=16 D=128 bf16 causal"}, "rows": rows}), flush=True)
        return
    if args.mode == "seqlen":
        rows = []
        for dtype in (torch.float32, torch.bfloat16):
            for Ts in range(256, 2049, 256):
                q, k1, k2, v1, v2, do = (t.to(dev) for t in make_inputs(2, 2, Ts, 64, dtype, seed=42))
                leaves = [t.clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
                kw = dict(softmax_scale=1 / 8, k1_window=24, k2_window=22, kk_left=None, kk_right=None, causal=True,
                          convert_to_float32=True)
                hold = {}

                def f():
                    with torch.no_grad():
                        return flash_trittention(q, k1, k2, v1, v2, **kw)

                def b():
                    hold["g"] = torch.autograd.grad(hold["o"], leaves, do, retain_graph=True)

                ms_f = time_events(f, 20, 5, torch)
                hold["o"] = flash_trittention(*leaves, **kw)
                ms_b = time_events(b, 20, 5, torch)
                nt = 4 * windowed_triples(Ts, 24, 22, Ts, Ts)
                rows.append({"dtype": str(dtype).split(".")[-1], "T": Ts, "fwd_ms": ms_f, "bwd_ms": ms_b,
                             "valid_triples": nt, "fwd_tflops": 4 * 64 * nt / ms_f / 1e9,
                             "bwd_tflops": 12 * 64 * nt / ms_b / 1e9})
        print(json.dumps({"metric": "triple-dot trittention fwd / bwd ms over T, windowed", "unit": "ms",
                          "config": {"workload": "triple-dot fwd+bwd B=2 H=2 D=64 causal, k1_window=24 k2_window=22, "
                                                 "convert_to_float32=True, T=256..2048"}, "rows": rows}), flush=True)
        return
    if args.mode == "published":
        # the reference's own forward table (h100/README.md:50-53, b200/README.md:53-56): milliseconds of its
        # best kernel on each machine; B=2 H=8 D=64 fp16 causal, softmax_scale 1/8
        cases = [(256, None, 0.298, 0.461), (512, None, 1.451, 2.111), (1024, None, 8.748, 11.61),
                 (2048, (128, 128, 32, 32), 1.163, 1.074)]
        rows = []
        for Ts, win, h100_ms, b200_ms in cases:
            ins = [t.to(dev) for t in make_inputs(2, 8, Ts, 64, torch.float16, seed=1, n=5)]
            w = win or (None, None, None, None)

            def f():
                with torch.no_grad():
                    return flash_trittention(*ins, softmax_scale=1 / 8, k1_window=w[0], k2_window=w[1], kk_left=w[2],
                                             kk_right=w[3], causal=True)

            ms = time_events(f, max(args.steps, 20), max(args.warmup, 5), torch)
            nt = 16 * (windowed_triples(Ts, *win) if win else triples(1, 1, Ts))
            rows.append({"T": Ts, "windows": win, "ms": ms, "tflops": 4 * 64 * nt / ms / 1e9,
                         "reference_h100_ms": h100_ms, "reference_b200_ms": b200_ms,
                         "speedup_vs_best_published": min(h100_ms, b200_ms) / ms})
        print(json.dumps({"metric": "triple-dot trittention fwd ms on the reference's published cases", "unit": "ms",
                          "config": {"workload": "triple-dot fwd B=2 H=8 D=64 fp16 causal"}, "rows": rows}), flush=True)
        return
    if args.mode == "dpsrange":
        rows = []
        for dtype in (torch.float32, torch.bfloat16):
            for Ts, kd in ((1024, None), (2048, 1024), (2048, 128), (4096, 2048), (4096, 128), (8192, 2048), (8192, 128)):
                r = dps_times(torch, dev, 1, 8, Ts, 64, 10, 3, dtype=dtype, k_diff=kd)
                rows.append({"dtype": str(dtype).split(".")[-1], "T": Ts, "k_diff": kd or Ts,
                             **{k: r[k] for k in ("fwd_ms", "bwd_ms", "executed_fwd_tflops", "executed_bwd_tflops",
                                                  "mfma_frac_fwd", "mfma_frac_bwd", "io_gbs_fwd", "io_gbs_bwd")}})
        print(json.dumps({"metric": "dot-product-sum trittention fwd / bwd ms", "unit": "ms",
                          "config": {"workload": "dot-product-sum fwd+bwd B=1 H=8 D=64 causal, T=1024..8192"},
                          "rows": rows}), flush=True)
        return
    if args.mode == "dps":
        ddtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype]
        r = dps_times(torch, dev, B, H, T, D, args.steps, args.warmup, dtype=ddtype)
        print(json.dumps({"metric": "dot-product-sum trittention fwd / bwd ms", "unit": "ms", **r}), flush=True)
        return
    tdtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype if args.mode == "tdp" else "bf16"]
    q, k1, k2, v1, v2, do = (t.to(dev) for t in make_inputs(B, H, T, D, tdtype, seed=0))
    leaves = [t.clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    kw = dict(softmax_scale=alpha, k1_window=None, k2_window=None, kk_left=None, kk_right=None, causal=True)
    if args.mode == "tdp" and args.convert:
        kw["convert_to_float32"] = True

    def fwd_only():
        with torch.no_grad():
            return flash_trittention(q, k1, k2, v1, v2, **kw)

    out_holder = {}

    def fwd_graph():
        out_holder["o"] = flash_trittention(*leaves, **kw)

    def bwd_only():  # the gradients are returned, not added into .grad (see dps_times)
        out_holder["g"] = torch.autograd.grad(out_holder["o"], leaves, do, retain_graph=True)

    def step():
        o = flash_trittention(*leaves, **kw)
        o.backward(do)

    n = triples(B, H, T)
    f_fwd, f_bwd = 4 * D * n, 12 * D * n

    if args.mode == "tdp":
        win = [int(x) for x in args.windows.split(",")] if args.windows else None
        if win:
            kw.update(k1_window=win[0], k2_window=win[1], kk_left=win[2], kk_right=win[3])
            n = B * H * windowed_triples(T, *win)
            f_fwd, f_bwd = 4 * D * n, 12 * D * n
        ms_fwd = time_events(fwd_only, args.steps, args.warmup, torch)
        fwd_graph()
        ms_bwd = time_events(bwd_only, args.steps, args.warmup, torch)
        print(json.dumps({"metric": "triple-dot trittention fwd / bwd", "unit": "ms", "fwd_ms": ms_fwd, "bwd_ms": ms_bwd,
                          "fwd_tflops": f_fwd / ms_fwd / 1e9, "bwd_tflops": f_bwd / ms_bwd / 1e9, "valid_triples": n,
                          "config": {"workload": f"triple-dot fwd+bwd B={B} H={H} T={T} D={D} {args.dtype} causal",
                                     "windows": win, "convert_to_float32": bool(args.convert)}}), flush=True)
        return

    if args.mode == "fwd":
        ms_fwd = time_events(fwd_only, args.steps, args.warmup, torch)
        print(json.dumps({"metric": "triple-dot trittention fwd TFLOP/s", "value": f_fwd / ms_fwd / 1e9,
                          "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "ms_per_step": ms_fwd, "frac_of_bf16_peak": f_fwd / ms_fwd / 1e9 / PEAK_BF16_TFLOPS,
                          "config": {"workload": f"triple-dot fwd B={B} H={H} T={T} D={D} bf16 causal"}}), flush=True)
        return

    # the timed region the driver's contract asks for: W warm-up steps, then exactly K steps
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    ms_fwd = time_events(fwd_only, max(args.steps, 5), 2, torch)
    fwd_graph()
    ms_bwd = time_events(bwd_only, max(args.steps // 2, 3), 1, torch)

    fwd_tf, bwd_tf = f_fwd / ms_fwd / 1e9, f_bwd / ms_bwd / 1e9
    default_workload = (B, H, T, D) == (4, 8, 1024, 64)
    probe = mfma_probe(torch, _lib)
    elem = 2
    bytes_fwd = 6 * B * H * T * D * elem + 4 * B * H * T
    bytes_bwd = 12 * B * H * T * D * elem + 8 * B * H * T
    props = torch.cuda.get_device_properties(0)
    result = {
        "metric": "triple-dot trittention fwd+bwd TFLOP/s (B=4 H=8 T=1024 D=64 bf16 causal)",
        "value": (f_fwd + f_bwd) / ms_step / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic N(0,1), seeded on the CPU, resident in HBM before timing",
        "config": {"workload": f"triple-dot fwd+bwd B={B} H={H} T={T} D={D} bf16 causal full-window",
                   "alpha": alpha, "valid_triples": n},
        "fwd_ms": ms_fwd, "bwd_ms": ms_bwd, "fwd_tflops": fwd_tf, "bwd_tflops": bwd_tf,
        "fwd_hbm_gbs": bytes_fwd / ms_fwd / 1e6, "bwd_hbm_gbs": bytes_bwd / ms_bwd / 1e6,
        "device": {"name": props.name, "cus": props.multi_processor_count,
                   "nominal_clock_mhz": nominal_clock_mhz(),
                   "peak_used": "2.5 PFLOP/s bf16 dense (256 CUs x 4096 flop/clk x 2.4 GHz nominal)",
                   # measured in this run: what a pure-MFMA kernel reaches, and the clock that implies
                   "mfma_probe": probe},
        # dominant kernel by time: the rows kernel of the backward, launched twice (dQ,dK2,dV2 then dK1,dU; the
        # first launch is tdp_bwd_rows_tile0_kernel, the same body with the 128 fp32 workgroups of query tile 0 in
        # its grid, the second tdp_bwd_rows_kernel).  Each launch is credited half of the backward's algorithmic
        # flops (6*D*N) and half of the event-timed backward (the prep/finish kernels in that time are < 1 %).
        "roofline": {"bound": "mfma",
                     "kernel": "tdp_bwd_rows_tile0_kernel<bf16,64,true> + tdp_bwd_rows_kernel<bf16,64,false> (the rows "
                               "kernel's two launches, averaged)",
                     "achieved": bwd_tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": bwd_tf / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BWD_ROWS if default_workload else None,
                     "traffic_source": TRAFFIC_SOURCE if default_workload else None,
                     "frac_of_sustained_mfma_rate": bwd_tf / probe["tflops"],
                     "flops_per_launch": f_bwd // 2, "ms_per_launch": ms_bwd / 2},
        "roofline_fwd": {"bound": "mfma", "kernel": "tdp_fwd_mfma_kernel<bf16,64,NT=2,8 waves>",
                         "achieved": fwd_tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": fwd_tf / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_FWD if default_workload else None,
                         "traffic_source": TRAFFIC_SOURCE if default_workload else None,
                         "frac_of_sustained_mfma_rate": fwd_tf / probe["tflops"],
                         "flops_per_launch": f_fwd, "ms_per_launch": ms_fwd},
    }
    if not args.brief:
        # the other BASELINE configurations, timed in the same run (parity for each: tests/test_gpu_*.py)
        short = max(5, min(args.steps, 20))
        result["other_configs"] = {
            "config1_tdp_fwd_fp32": tdp_times(torch, flash_trittention, dev, 1, 2, 64, 32, torch.float32, 20, 5,
                                              backward=False),
            "config2_tdp_fwd_bwd": tdp_times(torch, flash_trittention, dev, 2, 4, 256, 64, torch.bfloat16, 20, 5),
            # the headline shape as the reference's own scripts call it (convert_to_float32=True): the score
            # operands as hi + lo pairs on the same matrix-core kernels
            "config3_tdp_fwd_bwd_convert_to_float32": tdp_times(torch, flash_trittention, dev, 4, 8, 1024, 64,
                                                               torch.bfloat16, short, 2, convert=True),
            "config4_dps_fwd_bwd": dps_times(torch, dev, 4, 8, 1024, 64, 20, 5),
            "config5_tdp_fwd_sweep": {"workload": "triple-dot fwd B=1 H=16 D=128 bf16 causal",
                                      "rows": sweep_rows(torch, flash_trittention, dev, short)},
            "tdp_fwd_bwd_d128": tdp_times(torch, flash_trittention, dev, 4, 8, 1024, 128, torch.bfloat16, 3, 1),
            "tdp_fwd_bwd_fp32_d32": tdp_times(torch, flash_trittention, dev, 4, 8, 1024, 32, torch.float32, 2, 1),
        }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(T, D, alpha)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
