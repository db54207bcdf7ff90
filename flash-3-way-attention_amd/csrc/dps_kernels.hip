// Dot-product-sum trittention as two chained attention passes (O(T^2 D)).
//
//   exp(alpha (Q_q.K2_t + K1_s.K2_t)) = exp(alpha Q_q.K2_t) * exp(alpha K1_s.K2_t)
// and the mask (s <= t <= q, t - s <= k_diff) never couples s with q, so
//   inner:  lse1[t] = logsumexp_s alpha K1_s.K2_t,  R[t] = softmax_s(.) @ U,  W[t] = R[t] * V2[t]
//   outer:  O[q] = softmax_t(alpha Q_q.K2_t + lse1[t]) @ W,  LSE[q] = logsumexp_t(.)
// The backward is the two attention backwards chained through (dR, dlse1).
// Each output row has exactly one owner lane, so there are no atomics and
// results are bitwise reproducible.
//
// Kernels: one wave per workgroup, one lane per owned row; the rows of the
// other operand are staged through LDS and read as broadcasts.  All fp32.
#include "common.hpp"
#include "kernels.hpp"

namespace tritt {

constexpr int kRows = 32;  // staged rows per step

template <int D>
__device__ __forceinline__ void stage64(float (*dst)[D], const float* __restrict__ src, int row0, int T) {
    constexpr int kVec = D / 4;
    for (int i = threadIdx.x; i < kRows * kVec; i += 64) {
        int r = i / kVec, c = i % kVec;
        int row = min(row0 + r, T - 1);
        reinterpret_cast<float4*>(dst[r])[c] = reinterpret_cast<const float4*>(src + (size_t)row * D)[c];
    }
}

template <int D>
__device__ __forceinline__ float dotp(const float (&v)[D], const float* __restrict__ row) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
    for (int d = 0; d < D; d += 4) {
        float4 k = *reinterpret_cast<const float4*>(row + d);
        s0 = fmaf(v[d], k.x, s0);
        s1 = fmaf(v[d + 1], k.y, s1);
        s2 = fmaf(v[d + 2], k.z, s2);
        s3 = fmaf(v[d + 3], k.w, s3);
    }
    return (s0 + s1) + (s2 + s3);
}

template <int D>
__device__ __forceinline__ void axpy(float (&acc)[D], float p, const float* __restrict__ row) {
#pragma unroll
    for (int d = 0; d < D; d += 4) {
        float4 k = *reinterpret_cast<const float4*>(row + d);
        acc[d] = fmaf(p, k.x, acc[d]);
        acc[d + 1] = fmaf(p, k.y, acc[d + 1]);
        acc[d + 2] = fmaf(p, k.z, acc[d + 2]);
        acc[d + 3] = fmaf(p, k.w, acc[d + 3]);
    }
}

// valid pair (owner row r attends staged row a)
__device__ __forceinline__ bool pair_ok(int causal, int k_diff, int r, int a) {
    return !causal || ((a <= r) & (r - a <= k_diff));
}

// Attention forward with an optional per-key bias (log2 units).  Lane r owns row X[r].
//   out[r] = softmax_a(scale X[r].K[a] + bias[a]) @ V ;  lse_out[r] = lse_scale * log2-sum-exp2
//   out_mul[r] = out[r] * mul[r]   (when mul != nullptr)
template <int D>
__global__ __launch_bounds__(64) void attn_fwd_kernel(
    const float* __restrict__ X, const float* __restrict__ K, const float* __restrict__ V,
    const float* __restrict__ bias, const float* __restrict__ mul, float* __restrict__ out,
    float* __restrict__ out_mul, float* __restrict__ lse_out, float lse_scale, int T, float scale_log2,
    int causal, int k_diff) {
    __shared__ __align__(16) float sK[kRows][D];
    __shared__ __align__(16) float sV[kRows][D];
    __shared__ float sB[kRows];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; K += base; V += base;
    const int r0 = blockIdx.x * 64, r = r0 + threadIdx.x, rc = min(r, T - 1);
    const int r_hi = min(T - 1, r0 + 63);
    const int a_lo = causal ? max(0, r0 - k_diff) : 0, a_hi = causal ? r_hi : T - 1;

    float x[D], acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        x[d] = X[(size_t)rc * D + d] * scale_log2;
        acc[d] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int a0 = a_lo & ~(kRows - 1); a0 <= a_hi; a0 += kRows) {
        __syncthreads();
        stage64<D>(sK, K, a0, T);
        stage64<D>(sV, V, a0, T);
        if (threadIdx.x < kRows) sB[threadIdx.x] = bias ? bias[vbase + min(a0 + (int)threadIdx.x, T - 1)] : 0.f;
        __syncthreads();
        const int n = min(kRows, a_hi - a0 + 1);
        for (int aa = 0; aa < n; ++aa) {
            const int a = a0 + aa;
            if (r < T && pair_ok(causal, k_diff, r, a)) {
                const float s = dotp<D>(x, sK[aa]) + sB[aa];
                if (s > m) {
                    const float f = fast_exp2(m - s);
                    l *= f;
#pragma unroll
                    for (int d = 0; d < D; ++d) acc[d] *= f;
                    m = s;
                }
                const float p = fast_exp2(s - m);
                l += p;
                axpy<D>(acc, p, sV[aa]);
            }
        }
    }
    if (r < T) {
        const float inv = 1.0f / l;
#pragma unroll
        for (int d = 0; d < D; d += 4) {
            float4 o = make_float4(acc[d] * inv, acc[d + 1] * inv, acc[d + 2] * inv, acc[d + 3] * inv);
            *reinterpret_cast<float4*>(out + base + (size_t)r * D + d) = o;
            if (mul) {
                float4 mm = *reinterpret_cast<const float4*>(mul + base + (size_t)r * D + d);
                *reinterpret_cast<float4*>(out_mul + base + (size_t)r * D + d) =
                    make_float4(o.x * mm.x, o.y * mm.y, o.z * mm.z, o.w * mm.w);
            }
        }
        lse_out[vbase + r] = (m + fast_log2(l)) * lse_scale;
    }
}

// Attention backward, owner = query-like row r:
//   P = exp2(scale X[r].K[a] + bias[a] - lse2[r]);  dS = P (G[r].V[a] - delta[r]);
//   dX[r] = alpha * sum_a dS K[a]  (+ addend[r])
template <int D>
__global__ __launch_bounds__(64) void attn_bwd_row_kernel(
    const float* __restrict__ X, const float* __restrict__ G, const float* __restrict__ K,
    const float* __restrict__ V, const float* __restrict__ bias, const float* __restrict__ lse,
    float lse_to_log2, const float* __restrict__ delta, const float* __restrict__ addend,
    float* __restrict__ dX, int T, float alpha, int causal, int k_diff) {
    __shared__ __align__(16) float sK[kRows][D];
    __shared__ __align__(16) float sV[kRows][D];
    __shared__ float sB[kRows];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; G += base; K += base; V += base;
    const int r0 = blockIdx.x * 64, r = r0 + threadIdx.x, rc = min(r, T - 1);
    const int r_hi = min(T - 1, r0 + 63);
    const int a_lo = causal ? max(0, r0 - k_diff) : 0, a_hi = causal ? r_hi : T - 1;
    const float scale_log2 = alpha * kLog2e;

    float x[D], g[D], acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        x[d] = X[(size_t)rc * D + d] * scale_log2;
        g[d] = G[(size_t)rc * D + d];
        acc[d] = 0.f;
    }
    const float lse2 = lse[vbase + rc] * lse_to_log2, dl = delta[vbase + rc];
    for (int a0 = a_lo & ~(kRows - 1); a0 <= a_hi; a0 += kRows) {
        __syncthreads();
        stage64<D>(sK, K, a0, T);
        stage64<D>(sV, V, a0, T);
        if (threadIdx.x < kRows) sB[threadIdx.x] = bias ? bias[vbase + min(a0 + (int)threadIdx.x, T - 1)] : 0.f;
        __syncthreads();
        const int n = min(kRows, a_hi - a0 + 1);
        for (int aa = 0; aa < n; ++aa) {
            const int a = a0 + aa;
            if (r < T && pair_ok(causal, k_diff, r, a)) {
                const float s = dotp<D>(x, sK[aa]) + sB[aa];
                const float dp = dotp<D>(g, sV[aa]);
                axpy<D>(acc, fast_exp2(s - lse2) * (dp - dl), sK[aa]);
            }
        }
    }
    if (r < T) {
#pragma unroll
        for (int d = 0; d < D; d += 4) {
            float4 o = make_float4(acc[d] * alpha, acc[d + 1] * alpha, acc[d + 2] * alpha, acc[d + 3] * alpha);
            if (addend) {
                float4 e = *reinterpret_cast<const float4*>(addend + base + (size_t)r * D + d);
                o.x += e.x; o.y += e.y; o.z += e.z; o.w += e.w;
            }
            *reinterpret_cast<float4*>(dX + base + (size_t)r * D + d) = o;
        }
    }
}

// Attention backward, owner = key-like row a (the lane); the query-like rows r are staged:
//   dK[a] = alpha * sum_r dS X[r];  dV[a] = sum_r P G[r];  dbias[a] = sum_r dS
template <int D>
__global__ __launch_bounds__(64) void attn_bwd_col_kernel(
    const float* __restrict__ X, const float* __restrict__ G, const float* __restrict__ K,
    const float* __restrict__ V, const float* __restrict__ bias, const float* __restrict__ lse,
    float lse_to_log2, const float* __restrict__ delta, float* __restrict__ dK, float* __restrict__ dV,
    float* __restrict__ dbias, int T, float alpha, int causal, int k_diff) {
    __shared__ __align__(16) float sX[kRows][D];
    __shared__ __align__(16) float sG[kRows][D];
    __shared__ float sL[kRows], sD[kRows];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; G += base; K += base; V += base;
    const int c0 = blockIdx.x * 64, a = c0 + threadIdx.x, ac = min(a, T - 1);
    const int c_hi = min(T - 1, c0 + 63);
    const int r_lo = causal ? c0 : 0;
    const int r_hi = causal ? (int)min((long)T - 1, (long)c_hi + k_diff) : T - 1;
    const float scale_log2 = alpha * kLog2e;

    float k[D], v[D], accK[D], accV[D];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        k[d] = K[(size_t)ac * D + d] * scale_log2;
        v[d] = V[(size_t)ac * D + d];
        accK[d] = 0.f;
        accV[d] = 0.f;
    }
    const float b = bias ? bias[vbase + ac] : 0.f;
    float db = 0.f;
    for (int r0 = r_lo & ~(kRows - 1); r0 <= r_hi; r0 += kRows) {
        __syncthreads();
        stage64<D>(sX, X, r0, T);
        stage64<D>(sG, G, r0, T);
        if (threadIdx.x < kRows) {
            int rr = min(r0 + (int)threadIdx.x, T - 1);
            sL[threadIdx.x] = lse[vbase + rr] * lse_to_log2;
            sD[threadIdx.x] = delta[vbase + rr];
        }
        __syncthreads();
        const int n = min(kRows, r_hi - r0 + 1);
        for (int i = 0; i < n; ++i) {
            const int r = r0 + i;
            if (a < T && pair_ok(causal, k_diff, r, a)) {
                const float s = dotp<D>(k, sX[i]) + b;
                const float dp = dotp<D>(v, sG[i]);
                const float p = fast_exp2(s - sL[i]);
                const float ds = p * (dp - sD[i]);
                axpy<D>(accK, ds, sX[i]);
                axpy<D>(accV, p, sG[i]);
                db += ds;
            }
        }
    }
    if (a < T) {
#pragma unroll
        for (int d = 0; d < D; d += 4) {
            *reinterpret_cast<float4*>(dK + base + (size_t)a * D + d) =
                make_float4(accK[d] * alpha, accK[d + 1] * alpha, accK[d + 2] * alpha, accK[d + 3] * alpha);
            *reinterpret_cast<float4*>(dV + base + (size_t)a * D + d) =
                make_float4(accV[d], accV[d + 1], accV[d + 2], accV[d + 3]);
        }
        if (dbias) dbias[vbase + a] = db;
    }
}

// dV2 = dW * R;  dR = dW * V2;  delta1 = rowsum(dR * R) - dlse1   (one wave per row)
__global__ __launch_bounds__(256) void dps_mid_kernel(const float* __restrict__ dW, const float* __restrict__ R,
                                                      const float* __restrict__ V2, const float* __restrict__ dlse1,
                                                      float* __restrict__ dV2, float* __restrict__ dR,
                                                      float* __restrict__ delta1, int rows, int D) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    float part = 0.f;
    for (int d = lane; d < D; d += 64) {
        const size_t i = (size_t)row * D + d;
        const float dw = dW[i], r = R[i];
        const float dr = dw * V2[i];
        dV2[i] = dw * r;
        dR[i] = dr;
        part += dr * r;
    }
    part = wave_sum(part);
    if (lane == 0) delta1[row] = part - dlse1[row];
}

template <int D>
static hipError_t fwd_impl(const DpsArgs& a, hipStream_t st) {
    dim3 grid((a.T + 63) / 64, a.BH);
    const float sl2 = a.alpha * kLog2e;
    // inner: rows = K2[t], keys K1, values U; outputs R, W = R*V2, lse1 (log2 units)
    hipLaunchKernelGGL(attn_fwd_kernel<D>, grid, dim3(64), 0, st, a.k2, a.k1, a.u, (const float*)nullptr, a.v2,
                       a.r, a.w, a.lse1, 1.0f, a.T, sl2, a.causal, a.k_diff);
    // outer: rows = Q[q], keys K2 with bias lse1, values W; outputs O, LSE (natural log)
    hipLaunchKernelGGL(attn_fwd_kernel<D>, grid, dim3(64), 0, st, a.q, a.k2, a.w, (const float*)a.lse1,
                       (const float*)nullptr, a.o, (float*)nullptr, a.lse, kLn2, a.T, sl2, a.causal, a.T);
    return hipGetLastError();
}

template <int D>
static hipError_t bwd_impl(const DpsArgs& a, hipStream_t st) {
    dim3 grid((a.T + 63) / 64, a.BH);
    const float sl2 = a.alpha * kLog2e;
    const float* nobias = nullptr;
    // recompute the inner pass: R, W, lse1
    hipLaunchKernelGGL(attn_fwd_kernel<D>, grid, dim3(64), 0, st, a.k2, a.k1, a.u, nobias, a.v2, a.r, a.w, a.lse1,
                       1.0f, a.T, sl2, a.causal, a.k_diff);
    // outer pass: dQ ; (dK2 part, dW, dlse1)
    hipLaunchKernelGGL(attn_bwd_row_kernel<D>, grid, dim3(64), 0, st, a.q, a.d_o, a.k2, (const float*)a.w,
                       (const float*)a.lse1, (const float*)a.lse, kLog2e, a.delta, nobias, a.dq, a.T, a.alpha,
                       a.causal, a.T);
    hipLaunchKernelGGL(attn_bwd_col_kernel<D>, grid, dim3(64), 0, st, a.q, a.d_o, a.k2, (const float*)a.w,
                       (const float*)a.lse1, (const float*)a.lse, kLog2e, a.delta, a.dk2_part, a.dw, a.dlse1, a.T,
                       a.alpha, a.causal, a.T);
    const int rows = a.BH * a.T;
    hipLaunchKernelGGL(dps_mid_kernel, dim3((rows + 3) / 4), dim3(256), 0, st, (const float*)a.dw,
                       (const float*)a.r, a.v2, (const float*)a.dlse1, a.dv2, a.dr, a.delta1, rows, a.D);
    // inner pass: dK2 (total) ; (dK1, dU)
    hipLaunchKernelGGL(attn_bwd_row_kernel<D>, grid, dim3(64), 0, st, a.k2, (const float*)a.dr, a.k1, a.u, nobias,
                       (const float*)a.lse1, 1.0f, (const float*)a.delta1, (const float*)a.dk2_part, a.dk2, a.T,
                       a.alpha, a.causal, a.k_diff);
    hipLaunchKernelGGL(attn_bwd_col_kernel<D>, grid, dim3(64), 0, st, a.k2, (const float*)a.dr, a.k1, a.u, nobias,
                       (const float*)a.lse1, 1.0f, (const float*)a.delta1, a.dk1, a.du, (float*)nullptr, a.T,
                       a.alpha, a.causal, a.k_diff);
    return hipGetLastError();
}

hipError_t dps_fwd(const DpsArgs& a, hipStream_t st) {
    switch (a.D) {
        case 8: return fwd_impl<8>(a, st);
        case 16: return fwd_impl<16>(a, st);
        case 32: return fwd_impl<32>(a, st);
        case 64: return fwd_impl<64>(a, st);
        case 128: return fwd_impl<128>(a, st);
    }
    return hipErrorInvalidValue;
}

hipError_t dps_bwd(const DpsArgs& a, hipStream_t st) {
    switch (a.D) {
        case 8: return bwd_impl<8>(a, st);
        case 16: return bwd_impl<16>(a, st);
        case 32: return bwd_impl<32>(a, st);
        case 64: return bwd_impl<64>(a, st);
        case 128: return bwd_impl<128>(a, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace tritt
