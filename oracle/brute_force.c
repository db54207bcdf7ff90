/* Float64 brute-force restatement of the two trittention formulations.
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ (through ctypes) to pin
 * oracle/trittention_oracle.py; never linked into or called by the product.
 *
 * Plain triple loops over (q, j, k), one head at a time, no tiling, no
 * vectorisation.  Forward follows the equations of the reference's
 * README.md:13-37 and its naive modules
 *   triple_dot_product/trittention_pytorch.py:68-75 (mask), :81-101 (forward)
 *   dot_product_sum/trittention_pytorch.py:47-51 (mask), :56-81 (forward)
 * Gradients are the analytic ones (what autograd of those modules yields):
 *   Delta[q] = dO[q].O[q];  dP = dO[q].(U[j]*V2[k]);  dS = P (dP - Delta)
 * so that a sign, index or transposition slip in the PyTorch oracle (which
 * gets its gradients from autograd) shows up as a disagreement.
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC)
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

static double silu(double x) { return x / (1.0 + exp(-x)); }
static double dsilu(double x) {
    double s = 1.0 / (1.0 + exp(-x));
    return s * (1.0 + x * (1.0 - s));
}

/* triple-dot mask: 1 = masked out (trittention_pytorch.py:68-75) */
static int tdp_masked(int q, int j, int k, int causal, int k1w, int k2w, int kl, int kr) {
    if (!causal) return 0;
    return (j > q) || (k > q) || (q > j + k1w) || (q > k + k2w) || (j + kl < k) || (k + kr < j);
}

/* dot-product-sum mask, s = K1 row, t = K2 row (trittention_pytorch.py:47-51 by axis) */
static int dps_masked(int q, int s, int t, int causal, int k_diff) {
    if (!causal) return 0;
    return (s > t) || (t > q) || (t - s > k_diff);
}

/* variant 0: s = alpha sum_d Q K1 K2 ; variant 1: s = alpha (K2.Q + K1.K2) */
static double score(int variant, const double* q, const double* k1, const double* k2, int D, double alpha) {
    double acc = 0.0;
    if (variant == 0) {
        for (int d = 0; d < D; ++d) acc += q[d] * k1[d] * k2[d];
    } else {
        for (int d = 0; d < D; ++d) acc += k2[d] * (q[d] + k1[d]);
    }
    return alpha * acc;
}

/* One head.  All arrays row-major [T, D]; lse [T].  Gradient pointers may be
 * NULL (forward only).  w[0..3] = k1_window,k2_window,kk_left,kk_right for
 * variant 0;  w[0] = k_diff for variant 1. */
int trittention_brute(int variant, const double* Q, const double* K1, const double* K2,
                      const double* V1, const double* V2, const double* dO,
                      int T, int D, double alpha, int causal, const int* w,
                      double* O, double* LSE,
                      double* dQ, double* dK1, double* dK2, double* dV1, double* dV2) {
    double* U = (double*)malloc(sizeof(double) * T * D);
    double* dU = (double*)calloc((size_t)T * D, sizeof(double));
    if (!U || !dU) return -1;
    for (int i = 0; i < T * D; ++i) U[i] = silu(V1[i]);
    int grads = dQ && dK1 && dK2 && dV1 && dV2 && dO;
    if (grads) {
        memset(dQ, 0, sizeof(double) * T * D);
        memset(dK1, 0, sizeof(double) * T * D);
        memset(dK2, 0, sizeof(double) * T * D);
        memset(dV2, 0, sizeof(double) * T * D);
    }
#define MASKED(q, j, k) (variant == 0 ? tdp_masked(q, j, k, causal, w[0], w[1], w[2], w[3]) \
                                      : dps_masked(q, j, k, causal, w[0]))
    for (int q = 0; q < T; ++q) {
        /* pass 1: max, pass 2: sum, pass 3: output */
        double mx = -INFINITY;
        for (int j = 0; j < T; ++j)
            for (int k = 0; k < T; ++k) {
                if (MASKED(q, j, k)) continue;
                double s = score(variant, Q + q * D, K1 + j * D, K2 + k * D, D, alpha);
                if (s > mx) mx = s;
            }
        double sum = 0.0;
        for (int j = 0; j < T; ++j)
            for (int k = 0; k < T; ++k) {
                if (MASKED(q, j, k)) continue;
                sum += exp(score(variant, Q + q * D, K1 + j * D, K2 + k * D, D, alpha) - mx);
            }
        double lse = mx + log(sum);
        LSE[q] = lse;
        for (int d = 0; d < D; ++d) O[q * D + d] = 0.0;
        for (int j = 0; j < T; ++j)
            for (int k = 0; k < T; ++k) {
                if (MASKED(q, j, k)) continue;
                double p = exp(score(variant, Q + q * D, K1 + j * D, K2 + k * D, D, alpha) - lse);
                for (int d = 0; d < D; ++d) O[q * D + d] += p * U[j * D + d] * V2[k * D + d];
            }
        if (!grads) continue;
        double delta = 0.0;
        for (int d = 0; d < D; ++d) delta += dO[q * D + d] * O[q * D + d];
        for (int j = 0; j < T; ++j)
            for (int k = 0; k < T; ++k) {
                if (MASKED(q, j, k)) continue;
                double p = exp(score(variant, Q + q * D, K1 + j * D, K2 + k * D, D, alpha) - lse);
                double dp = 0.0;
                for (int d = 0; d < D; ++d) dp += dO[q * D + d] * U[j * D + d] * V2[k * D + d];
                double ds = p * (dp - delta);
                for (int d = 0; d < D; ++d) {
                    double qd = Q[q * D + d], k1d = K1[j * D + d], k2d = K2[k * D + d];
                    if (variant == 0) {
                        dQ[q * D + d] += alpha * ds * k1d * k2d;
                        dK1[j * D + d] += alpha * ds * qd * k2d;
                        dK2[k * D + d] += alpha * ds * qd * k1d;
                    } else {
                        dQ[q * D + d] += alpha * ds * k2d;
                        dK1[j * D + d] += alpha * ds * k2d;
                        dK2[k * D + d] += alpha * ds * (qd + k1d);
                    }
                    dU[j * D + d] += p * dO[q * D + d] * V2[k * D + d];
                    dV2[k * D + d] += p * dO[q * D + d] * U[j * D + d];
                }
            }
    }
#undef MASKED
    if (grads)
        for (int i = 0; i < T * D; ++i) dV1[i] = dU[i] * dsilu(V1[i]);
    free(U);
    free(dU);
    return 0;
}
