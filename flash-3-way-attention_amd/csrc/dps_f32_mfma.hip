// Dot-product-sum trittention for fp32 tensors on the matrix cores (v_mfma_f32_32x32x2_f32), D = 32 or 64.
//
// The same two chained attention passes as dps_kernels.hip (inner: lse1, R = softmax_s(alpha K1_s.K2_t) @ U;
// outer: softmax_t(alpha Q_q.K2_t + lse1[t]) @ (R * V2); backward = the two attention backwards chained through
// dR and dlse1) and the same three kernels with the same arguments, "attention with a per-key bias" forward,
// backward by owner rows and backward by owner columns; only the products run on the fp32 MFMA instead of one
// lane per row on the vector ALUs.  True fp32 operands, products and accumulation (the 1e-4 bar of fp32 tensors).
//
// Tiling.  A workgroup = two waves = 64 owner rows (32 per wave, one per MFMA column = lane % 32); the other
// operand's rows stream through LDS in 32-row tiles shared by the two waves (fetched into registers one tile
// ahead, row stride D + 1 floats).  A 32x32 score tile is D / 2 MFMAs with the contraction split by lane half:
//   S^T[a, r] = sum_ks  Ka[a][g D/2 + ks] * Xr[r][g D/2 + ks]        (A from LDS, B from the owner's registers)
// It leaves the MFMA with lane <-> owner row and registers <-> streamed rows (row c_row(g, i) in register i), which
// is the B-operand layout of the output products
//   O^T[d, r] += sum_a V^T[d, a] P^T[a, r]                            (A from LDS, B = the P registers)
// so P never moves between lanes and every per-owner quantity (running maximum, sums, LSE, Delta) is lane-local.
// One owner per output element: no atomics, bitwise reproducible.
#include "common.hpp"
#include "kernels.hpp"
#include "mfma.hpp"

namespace tritt {
namespace {

__device__ __forceinline__ f32x16 mma2(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

constexpr int kOwnerRows = 64;  // per workgroup

// valid pair (owner-like row r attends key-like row a)
__device__ __forceinline__ bool pair_valid(int causal, int k_diff, int r, int a) {
    return !causal || ((a <= r) & (r - a <= k_diff));
}

// Two 32 x D fp32 tiles (rows row0 .. row0 + 31 of A and of B, clamped to T - 1) through registers into LDS.
template <int D>
struct Stage2 {
    static constexpr int kPer = 32 * D / 4 / 128;  // float4 pieces per thread and tensor
    float4 a[kPer], b[kPer];
};
template <int D>
__device__ __forceinline__ void stage_fetch2(Stage2<D>& s, const float* __restrict__ A, const float* __restrict__ B,
                                             int row0, int T) {
    constexpr int kVec = D / 4;
#pragma unroll
    for (int i = 0; i < Stage2<D>::kPer; ++i) {
        const int idx = threadIdx.x + i * 128, row = min(row0 + idx / kVec, T - 1), c = idx % kVec;
        s.a[i] = *reinterpret_cast<const float4*>(A + (size_t)row * D + c * 4);
        s.b[i] = *reinterpret_cast<const float4*>(B + (size_t)row * D + c * 4);
    }
}
template <int D>
__device__ __forceinline__ void stage_store2(const Stage2<D>& s, float* sA, float* sB) {
    constexpr int kVec = D / 4, LD = D + 1;
#pragma unroll
    for (int i = 0; i < Stage2<D>::kPer; ++i) {
        const int idx = threadIdx.x + i * 128, row = idx / kVec, c = idx % kVec;
        float* pa = sA + row * LD + c * 4;
        float* pb = sB + row * LD + c * 4;
        pa[0] = s.a[i].x; pa[1] = s.a[i].y; pa[2] = s.a[i].z; pa[3] = s.a[i].w;
        pb[0] = s.b[i].x; pb[1] = s.b[i].y; pb[2] = s.b[i].z; pb[3] = s.b[i].w;
    }
}

// With one or two waves per SIMD a chain of MFMAs that accumulate into one tile waits for each result in turn, so
// every loop below walks two independent accumulators alternately.
// S^T tile: rows = the 32 staged rows, columns = the wave's owner rows; `own` = the owner's operand registers
template <int D>
__device__ __forceinline__ f32x16 score_tile(const float* sT, const float (&own)[D / 2], int n, int g) {
    constexpr int KS = D / 2, LD = D + 1;
    f32x16 s, t;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        s[i] = 0.f;
        t[i] = 0.f;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks += 2) {
        s = mma2(sT[n * LD + g * KS + ks], own[ks], s);
        t = mma2(sT[n * LD + g * KS + ks + 1], own[ks + 1], t);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] += t[i];
    return s;
}
// two score tiles at once (S from sA / ownA, dP from sB / ownB)
template <int D>
__device__ __forceinline__ void score_tiles(const float* sA, const float (&ownA)[D / 2], const float* sB,
                                            const float (&ownB)[D / 2], f32x16& s, f32x16& dp, int n, int g) {
    constexpr int KS = D / 2, LD = D + 1;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        s[i] = 0.f;
        dp[i] = 0.f;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        s = mma2(sA[n * LD + g * KS + ks], ownA[ks], s);
        dp = mma2(sB[n * LD + g * KS + ks], ownB[ks], dp);
    }
}
// acc^T[d, owner] += sum over the staged rows of T^T[d, row] * w[row, owner]   (w in score-tile layout)
template <int D>
__device__ __forceinline__ void output_tile(f32x16 (&acc)[D / 32], const float* sT, const f32x16& w, int n, int g) {
    constexpr int LD = D + 1, DT = D / 32;
    if constexpr (DT == 1) {  // one column tile: split the staged rows over two accumulators
        f32x16 t;
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            acc[0] = mma2(sT[c_row(g, i) * LD + n], w[i], acc[0]);
            t = mma2(sT[c_row(g, i + 1) * LD + n], w[i + 1], t);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[0][i] += t[i];
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc[dt] = mma2(sT[c_row(g, i) * LD + dt * 32 + n], w[i], acc[dt]);
    }
}
// two output products at once
template <int D>
__device__ __forceinline__ void output_tiles(f32x16 (&accA)[D / 32], const float* sA, const f32x16& wa,
                                             f32x16 (&accB)[D / 32], const float* sB, const f32x16& wb, int n, int g) {
    constexpr int LD = D + 1, DT = D / 32;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            accA[dt] = mma2(sA[c_row(g, i) * LD + dt * 32 + n], wa[i], accA[dt]);
            accB[dt] = mma2(sB[c_row(g, i) * LD + dt * 32 + n], wb[i], accB[dt]);
        }
}

// heavy-first tile order under a causal mask (the last owner tiles stream the most rows)
__device__ __forceinline__ int owner_tile(int causal) { return causal ? gridDim.x - 1 - blockIdx.x : blockIdx.x; }

// Attention forward with an optional per-key bias (log2 units):
//   out[r] = softmax_a(scale X[r].K[a] + bias[a]) @ V ;  lse_out[r] = lse_scale * log2-sum-exp2
//   out_mul[r] = out[r] * mul[r]   (when mul != nullptr)
template <int D>
__global__ __launch_bounds__(128, 2) void attn_fwd_f32m_kernel(
    const float* __restrict__ X, const float* __restrict__ K, const float* __restrict__ V,
    const float* __restrict__ bias, const float* __restrict__ mul, float* __restrict__ out,
    float* __restrict__ out_mul, float* __restrict__ lse_out, float lse_scale, int T, float scale_log2, int causal,
    int k_diff) {
    constexpr int DT = D / 32, KS = D / 2, LD = D + 1;
    __shared__ float sK[32 * LD], sV[32 * LD], sBias[32];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; K += base; V += base;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5, wave = tid >> 6;
    const int r0 = owner_tile(causal) * kOwnerRows, r = r0 + wave * 32 + n, rc = min(r, T - 1);
    const int r_hi = min(T - 1, r0 + kOwnerRows - 1);
    const int a_lo = causal ? max(0, r0 - k_diff) : 0, a_hi = causal ? r_hi : T - 1;
    // this wave's owner rows and the staged rows they can reach
    const int wr_lo = r0 + wave * 32, wr_hi = min(T - 1, wr_lo + 31);

    float x[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) x[ks] = X[(size_t)rc * D + g * KS + ks] * scale_log2;
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    Stage2<D> st;
    const int a_first = a_lo & ~31;
    stage_fetch2<D>(st, K, V, a_first, T);
    for (int a0 = a_first; a0 <= a_hi; a0 += 32) {
        __syncthreads();
        stage_store2<D>(st, sK, sV);
        if (tid < 32) sBias[tid] = bias ? bias[vbase + min(a0 + tid, T - 1)] : 0.f;
        __syncthreads();
        if (a0 + 32 <= a_hi) stage_fetch2<D>(st, K, V, a0 + 32, T);
        if (wr_lo >= T) continue;  // a wave with no row inside the sequence (ragged last tile)
        if (causal && (a0 > wr_hi || a0 + 31 < wr_lo - k_diff)) continue;  // nothing in reach of this wave
        f32x16 s = score_tile<D>(sK, x, n, g);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int a = a0 + c_row(g, i);
            const bool ok = (a < T) & (r < T) & pair_valid(causal, k_diff, r, a);
            s[i] = ok ? s[i] + sBias[c_row(g, i)] : -INFINITY;
            mx = fmaxf(mx, s[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float f = m_new == -INFINITY ? 1.f : fast_exp2(m - m_new);  // nothing seen yet: keep the zeros
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = s[i] == -INFINITY ? 0.f : fast_exp2(s[i] - m_new);
            ps += s[i];
        }
        ps += __shfl_xor(ps, 32, 64);
        l = l * f + ps;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[dt][i] *= f;
        output_tile<D>(acc, sV, s, n, g);
    }
    if (r < T) {
        const float inv = 1.0f / l;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                // registers 4 i4 .. 4 i4 + 3 are four consecutive columns d of row r
                const size_t off = base + (size_t)r * D + dt * 32 + c_row(g, i4 * 4);
                const float4 o = make_float4(acc[dt][i4 * 4] * inv, acc[dt][i4 * 4 + 1] * inv, acc[dt][i4 * 4 + 2] * inv,
                                             acc[dt][i4 * 4 + 3] * inv);
                *reinterpret_cast<float4*>(out + off) = o;
                if (mul) {
                    const float4 mm = *reinterpret_cast<const float4*>(mul + off);
                    *reinterpret_cast<float4*>(out_mul + off) = make_float4(o.x * mm.x, o.y * mm.y, o.z * mm.z, o.w * mm.w);
                }
            }
        if (g == 0) lse_out[vbase + r] = (m + fast_log2(l)) * lse_scale;
    }
}

// Attention backward, owner = query-like row r:
//   P = exp2(scale X[r].K[a] + bias[a] - lse2[r]);  dS = P (G[r].V[a] - delta[r]);
//   dX[r] = alpha * sum_a dS K[a]  (+ addend[r])
template <int D>
__global__ __launch_bounds__(128, 2) void attn_bwd_row_f32m_kernel(
    const float* __restrict__ X, const float* __restrict__ G, const float* __restrict__ K,
    const float* __restrict__ V, const float* __restrict__ bias, const float* __restrict__ lse, float lse_to_log2,
    const float* __restrict__ delta, const float* __restrict__ addend, float* __restrict__ dX, int T, float alpha,
    int causal, int k_diff) {
    constexpr int DT = D / 32, KS = D / 2, LD = D + 1;
    __shared__ float sK[32 * LD], sV[32 * LD], sBias[32];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; G += base; K += base; V += base;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5, wave = tid >> 6;
    const int r0 = owner_tile(causal) * kOwnerRows, r = r0 + wave * 32 + n, rc = min(r, T - 1);
    const int r_hi = min(T - 1, r0 + kOwnerRows - 1);
    const int a_lo = causal ? max(0, r0 - k_diff) : 0, a_hi = causal ? r_hi : T - 1;
    const int wr_lo = r0 + wave * 32, wr_hi = min(T - 1, wr_lo + 31);
    const float scale_log2 = alpha * kLog2e;

    float x[KS], gg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        x[ks] = X[(size_t)rc * D + g * KS + ks] * scale_log2;
        gg[ks] = G[(size_t)rc * D + g * KS + ks];
    }
    const float lse2 = lse[vbase + rc] * lse_to_log2, dl = delta[vbase + rc];
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

    Stage2<D> st;
    const int a_first = a_lo & ~31;
    stage_fetch2<D>(st, K, V, a_first, T);
    for (int a0 = a_first; a0 <= a_hi; a0 += 32) {
        __syncthreads();
        stage_store2<D>(st, sK, sV);
        if (tid < 32) sBias[tid] = bias ? bias[vbase + min(a0 + tid, T - 1)] : 0.f;
        __syncthreads();
        if (a0 + 32 <= a_hi) stage_fetch2<D>(st, K, V, a0 + 32, T);
        if (wr_lo >= T) continue;
        if (causal && (a0 > wr_hi || a0 + 31 < wr_lo - k_diff)) continue;
        f32x16 s, dp;
        score_tiles<D>(sK, x, sV, gg, s, dp, n, g);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int a = a0 + c_row(g, i);
            const bool ok = (a < T) & (r < T) & pair_valid(causal, k_diff, r, a);
            s[i] = ok ? fast_exp2(s[i] + sBias[c_row(g, i)] - lse2) * (dp[i] - dl) : 0.f;
        }
        output_tile<D>(acc, sK, s, n, g);
    }
    if (r < T) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const size_t off = base + (size_t)r * D + dt * 32 + c_row(g, i4 * 4);
                float4 o = make_float4(acc[dt][i4 * 4] * alpha, acc[dt][i4 * 4 + 1] * alpha, acc[dt][i4 * 4 + 2] * alpha,
                                       acc[dt][i4 * 4 + 3] * alpha);
                if (addend) {
                    const float4 e = *reinterpret_cast<const float4*>(addend + off);
                    o.x += e.x; o.y += e.y; o.z += e.z; o.w += e.w;
                }
                *reinterpret_cast<float4*>(dX + off) = o;
            }
    }
}

// Attention backward, owner = key-like row a (the MFMA column); the query-like rows r are staged:
//   dK[a] = alpha * sum_r dS X[r];  dV[a] = sum_r P G[r];  dbias[a] = sum_r dS
template <int D>
__global__ __launch_bounds__(128, (D <= 32 ? 2 : 1)) void attn_bwd_col_f32m_kernel(
    const float* __restrict__ X, const float* __restrict__ G, const float* __restrict__ K,
    const float* __restrict__ V, const float* __restrict__ bias, const float* __restrict__ lse, float lse_to_log2,
    const float* __restrict__ delta, float* __restrict__ dK, float* __restrict__ dV, float* __restrict__ dbias, int T,
    float alpha, int causal, int k_diff) {
    constexpr int DT = D / 32, KS = D / 2, LD = D + 1;
    __shared__ float sX[32 * LD], sG[32 * LD], sL[32], sD[32];
    const size_t base = (size_t)blockIdx.y * T * D, vbase = (size_t)blockIdx.y * T;
    X += base; G += base; K += base; V += base;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5, wave = tid >> 6;
    // heavy first: under a causal mask the FIRST owner columns see the most rows
    const int c0 = blockIdx.x * kOwnerRows, a = c0 + wave * 32 + n, ac = min(a, T - 1);
    const int c_hi = min(T - 1, c0 + kOwnerRows - 1);
    const int r_lo = causal ? c0 : 0;
    const int r_hi = causal ? (int)min((long)T - 1, (long)c_hi + k_diff) : T - 1;
    const int wa_lo = c0 + wave * 32, wa_hi = min(T - 1, wa_lo + 31);
    const float scale_log2 = alpha * kLog2e;

    float k[KS], v[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        k[ks] = K[(size_t)ac * D + g * KS + ks] * scale_log2;
        v[ks] = V[(size_t)ac * D + g * KS + ks];
    }
    const float b = bias ? bias[vbase + ac] : 0.f;
    f32x16 accK[DT], accV[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            accK[dt][i] = 0.f;
            accV[dt][i] = 0.f;
        }
    float db = 0.f;

    Stage2<D> st;
    const int r_first = r_lo & ~31;
    stage_fetch2<D>(st, X, G, r_first, T);
    for (int rr0 = r_first; rr0 <= r_hi; rr0 += 32) {
        __syncthreads();
        stage_store2<D>(st, sX, sG);
        if (tid < 32) {
            const int rr = min(rr0 + tid, T - 1);
            sL[tid] = lse[vbase + rr] * lse_to_log2;
            sD[tid] = delta[vbase + rr];
        }
        __syncthreads();
        if (rr0 + 32 <= r_hi) stage_fetch2<D>(st, X, G, rr0 + 32, T);
        if (wa_lo >= T) continue;
        if (causal && (rr0 + 31 < wa_lo || (long)rr0 > (long)wa_hi + k_diff)) continue;  // nothing in reach
        f32x16 s, dp;  // rows = staged r, columns = owner a
        score_tiles<D>(sX, k, sG, v, s, dp, n, g);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int rr = rr0 + c_row(g, i);
            const bool ok = (rr < T) & (a < T) & pair_valid(causal, k_diff, rr, a);
            const float p = ok ? fast_exp2(s[i] + b - sL[c_row(g, i)]) : 0.f;
            const float ds = p * (dp[i] - sD[c_row(g, i)]);
            s[i] = ds;
            dp[i] = p;
            db += ds;
        }
        output_tiles<D>(accK, sX, s, accV, sG, dp, n, g);
    }
    db += __shfl_xor(db, 32, 64);
    if (a < T) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const size_t off = base + (size_t)a * D + dt * 32 + c_row(g, i4 * 4);
                *reinterpret_cast<float4*>(dK + off) = make_float4(accK[dt][i4 * 4] * alpha, accK[dt][i4 * 4 + 1] * alpha,
                                                                   accK[dt][i4 * 4 + 2] * alpha, accK[dt][i4 * 4 + 3] * alpha);
                *reinterpret_cast<float4*>(dV + off) = make_float4(accV[dt][i4 * 4], accV[dt][i4 * 4 + 1], accV[dt][i4 * 4 + 2],
                                                                   accV[dt][i4 * 4 + 3]);
            }
        if (dbias && g == 0) dbias[vbase + a] = db;
    }
}

// dV2 = dW * R;  dR = dW * V2;  delta1 = rowsum(dR * R) - dlse1   (one wave per row)
__global__ __launch_bounds__(256) void dps_mid_f32m_kernel(const float* __restrict__ dW, const float* __restrict__ R,
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
hipError_t fwd_impl(const DpsArgs& a, hipStream_t st) {
    const dim3 grid((a.T + kOwnerRows - 1) / kOwnerRows, a.BH);
    const float sl2 = a.alpha * kLog2e;
    // inner: rows = K2[t], keys K1, values U; outputs R, W = R * V2, lse1 (log2 units)
    hipLaunchKernelGGL(attn_fwd_f32m_kernel<D>, grid, dim3(128), 0, st, a.k2, a.k1, a.u, (const float*)nullptr, a.v2,
                       a.r, a.w, a.lse1, 1.0f, a.T, sl2, a.causal, a.k_diff);
    // outer: rows = Q[q], keys K2 with bias lse1, values W; outputs O, LSE (natural log)
    hipLaunchKernelGGL(attn_fwd_f32m_kernel<D>, grid, dim3(128), 0, st, a.q, a.k2, (const float*)a.w,
                       (const float*)a.lse1, (const float*)nullptr, a.o, (float*)nullptr, a.lse, kLn2, a.T, sl2,
                       a.causal, a.T);
    return hipGetLastError();
}

template <int D>
hipError_t bwd_impl(const DpsArgs& a, hipStream_t st) {
    const dim3 grid((a.T + kOwnerRows - 1) / kOwnerRows, a.BH);
    const float sl2 = a.alpha * kLog2e;
    const float* nobias = nullptr;
    // recompute the inner pass: R, W, lse1
    hipLaunchKernelGGL(attn_fwd_f32m_kernel<D>, grid, dim3(128), 0, st, a.k2, a.k1, a.u, nobias, a.v2, a.r, a.w, a.lse1,
                       1.0f, a.T, sl2, a.causal, a.k_diff);
    // outer pass: dQ ; (dK2 part, dW, dlse1)
    hipLaunchKernelGGL(attn_bwd_row_f32m_kernel<D>, grid, dim3(128), 0, st, a.q, a.d_o, a.k2, (const float*)a.w,
                       (const float*)a.lse1, (const float*)a.lse, kLog2e, a.delta, nobias, a.dq, a.T, a.alpha, a.causal,
                       a.T);
    hipLaunchKernelGGL(attn_bwd_col_f32m_kernel<D>, grid, dim3(128), 0, st, a.q, a.d_o, a.k2, (const float*)a.w,
                       (const float*)a.lse1, (const float*)a.lse, kLog2e, a.delta, a.dk2_part, a.dw, a.dlse1, a.T,
                       a.alpha, a.causal, a.T);
    const int rows = a.BH * a.T;
    hipLaunchKernelGGL(dps_mid_f32m_kernel, dim3((rows + 3) / 4), dim3(256), 0, st, (const float*)a.dw,
                       (const float*)a.r, a.v2, (const float*)a.dlse1, a.dv2, a.dr, a.delta1, rows, a.D);
    // inner pass: dK2 (total) ; (dK1, dU)
    hipLaunchKernelGGL(attn_bwd_row_f32m_kernel<D>, grid, dim3(128), 0, st, a.k2, (const float*)a.dr, a.k1, a.u, nobias,
                       (const float*)a.lse1, 1.0f, (const float*)a.delta1, (const float*)a.dk2_part, a.dk2, a.T, a.alpha,
                       a.causal, a.k_diff);
    hipLaunchKernelGGL(attn_bwd_col_f32m_kernel<D>, grid, dim3(128), 0, st, a.k2, (const float*)a.dr, a.k1, a.u, nobias,
                       (const float*)a.lse1, 1.0f, (const float*)a.delta1, a.dk1, a.du, (float*)nullptr, a.T, a.alpha,
                       a.causal, a.k_diff);
    return hipGetLastError();
}

}  // namespace

bool f32_mfma_dps_supported(int D) { return D == 32 || D == 64; }

hipError_t f32_mfma_dps_fwd(const DpsArgs& a, hipStream_t st) {
    if (a.D == 32) return fwd_impl<32>(a, st);
    if (a.D == 64) return fwd_impl<64>(a, st);
    return hipErrorInvalidValue;
}
hipError_t f32_mfma_dps_bwd(const DpsArgs& a, hipStream_t st) {
    if (a.D == 32) return bwd_impl<32>(a, st);
    if (a.D == 64) return bwd_impl<64>(a, st);
    return hipErrorInvalidValue;
}

}  // namespace tritt
