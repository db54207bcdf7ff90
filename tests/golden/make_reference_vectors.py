#!/usr/bin/env python3
"""Writes tests/golden/windowed_masks.npz: inputs, outputs and input gradients of the reference's
two naive (dense, CPU-runnable) modules on tiny windowed cases.

These vectors pin the one thing mathematics does not fix about the oracle: the axis conventions
of the window parameters (k1_window, k2_window, kk_left, kk_right for the triple-dot variant,
k_diff for the dot-product-sum variant).  Run in the build container only; needs the reference
checkout at /root/reference (never available where the GPU tests run).

    python tests/golden/make_reference_vectors.py
"""
import os
import sys

import numpy as np
import torch

REF_SRC = "/root/reference/src"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "windowed_masks.npz")

TDP_CASES = [  # (causal, k1_window, k2_window, kk_left, kk_right)
    (True, None, None, None, None),
    (True, 3, 5, 2, 1),
    (True, 0, 0, 0, 0),
    (True, None, 2, None, 0),
    (True, 4, None, 1, None),
    (True, 1, 7, 0, 3),
    (False, 3, 5, 2, 1),
]
DPS_CASES = [(True, 1024), (True, 0), (True, 2), (True, 5)]  # (causal, k_diff)
B, H, T, D = 1, 1, 12, 16


def main():
    sys.path.insert(0, REF_SRC)
    from flash_trittention.triple_dot_product.trittention_pytorch import Trittention_pytorch as NaiveTdp
    from flash_trittention.dot_product_sum.trittention_pytorch import Trittention_pytorch as NaiveDps

    g = torch.Generator().manual_seed(20240607)
    # fp32-representable values, evaluated by the reference module in float64
    base = [torch.randn(B, H, T, D, generator=g, dtype=torch.float32).double() for _ in range(6)]
    alpha = 0.5
    out = {"alpha": np.float64(alpha), "shape": np.array([B, H, T, D])}
    for name, t in zip(("q", "k1", "k2", "v1", "v2", "d_o"), base):
        out[name] = t.numpy().astype(np.float32)

    def run(module, tag):
        leaves = [t.clone().requires_grad_(True) for t in base[:5]]
        res = module(*leaves)
        z = res[0]
        # the modules' auxiliary returns (pre-softmax scores, gated values, M and, for triple-dot, L): they pin
        # the return tuples of the oracle's drop-in Trittention_pytorch classes
        for name, t in zip(("pre", "vgated", "M", "L"), res[1:]):
            out[f"{tag}_{name}"] = t.detach().numpy().copy()
        z.backward(base[5])
        out[tag + "_o"] = z.detach().numpy()
        for n, t in zip(("dq", "dk1", "dk2", "dv1", "dv2"), leaves):
            out[f"{tag}_{n}"] = t.grad.numpy()

    for i, (causal, k1w, k2w, kl, kr) in enumerate(TDP_CASES):
        m = NaiveTdp(causal=causal, softmax_scale=alpha, n_ctx=16, k1_window=k1w, k2_window=k2w,
                     kk_left=kl, kk_right=kr)
        run(m, f"tdp{i}")
        out[f"tdp{i}_cfg"] = np.array([int(causal)] + [-1 if w is None else w for w in (k1w, k2w, kl, kr)])
    for i, (causal, k_diff) in enumerate(DPS_CASES):
        m = NaiveDps(causal=causal, softmax_scale=alpha, n_ctx=16, k_diff=k_diff)
        run(m, f"dps{i}")
        out[f"dps{i}_cfg"] = np.array([int(causal), k_diff])
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
