// fp32 VALU kernels for triple-dot-product trittention: the full-precision
// path (fp32 tensors, windowed masks, any T).  Every lane owns one "virtual
// query row" (q, b): the vector Q[q] * K[b] is kept in registers and is
// contracted against rows of the other key tensor that are staged in LDS and
// read as wave-wide broadcasts, so the inner loop is pure FMA work with an
// ordinary (FlashAttention-style) online softmax per lane; the rows of one
// query are merged across lanes once per 64-wide tile of b.
//
// All tensors here are fp32 [BH, T, D]; other element types are converted to
// fp32 scratch copies by the caller (see capi.hip).  U = SiLU(V1).
#include "common.hpp"
#include "kernels.hpp"

namespace tritt {

constexpr int kStageRows = 32;

template <int D>
__device__ __forceinline__ void stage_rows(float (*dst)[D], const float* __restrict__ src, int row0, int T) {
    // 256 threads copy kStageRows x D floats; rows past the end are clamped (their values are
    // never used: the callers mask by index).
    constexpr int kVec = D / 4;
    for (int i = threadIdx.x; i < kStageRows * kVec; i += 256) {
        int r = i / kVec, c = i % kVec;
        int row = min(row0 + r, T - 1);
        reinterpret_cast<float4*>(dst[r])[c] = reinterpret_cast<const float4*>(src + (size_t)row * D)[c];
    }
}

template <int D>
__device__ __forceinline__ float dot_lds(const float (&v)[D], const float* __restrict__ row) {
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
__device__ __forceinline__ void axpy_lds(float (&acc)[D], float p, const float* __restrict__ row) {
#pragma unroll
    for (int d = 0; d < D; d += 4) {
        float4 k = *reinterpret_cast<const float4*>(row + d);
        acc[d] = fmaf(p, k.x, acc[d]);
        acc[d + 1] = fmaf(p, k.y, acc[d + 1]);
        acc[d + 2] = fmaf(p, k.z, acc[d + 2]);
        acc[d + 3] = fmaf(p, k.w, acc[d + 3]);
    }
}

// The backward kernels hold four D-vectors per virtual row; beyond D = 64 that no longer fits one
// lane's registers, so a row is shared by LP = D/64 lanes, each owning DL = D/LP consecutive
// columns: a wave then sweeps RPT = 64/LP rows at a time and the two partial dot products of a
// row meet through one cross-lane add.
template <int D>
struct RowSplit {
    static constexpr int LP = D > 64 ? D / 64 : 1;
    static constexpr int DL = D / LP;
    static constexpr int RPT = 64 / LP;
    static_assert(LP <= 2, "one or two lanes per row");
};
// sum over the lanes that hold the same column part (all 64, or the 32 of one half)
template <int LP>
__device__ __forceinline__ float part_sum(float v) {
#pragma unroll
    for (int off = 32 / LP; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
template <int LP>
__device__ __forceinline__ float join_parts(float v) {
    if constexpr (LP == 2) v += __shfl_xor(v, 32, 64);
    return v;
}

// ------------------------------------------------------------------------------------------
// Forward.  grid = (ceil(T/4), BH), 256 threads: wave w owns query q = 4*blockIdx.x + w, its
// lanes sweep the owner index b (K2/V2 rows) in tiles of 64; staged index a = K1/U rows.
template <int D>
__global__ __launch_bounds__(256) void tdp_fwd_generic_kernel(
    const float* __restrict__ Q, const float* __restrict__ KA, const float* __restrict__ KB,
    const float* __restrict__ VA, const float* __restrict__ VB, float* __restrict__ O,
    float* __restrict__ LSE, int T, float scale_log2, TdpMask mask) {
    __shared__ __align__(16) float sK[kStageRows][D];
    __shared__ __align__(16) float sV[kStageRows][D];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t base = (size_t)blockIdx.y * T * D;
    Q += base; KA += base; KB += base; VA += base; VB += base; O += base;
    LSE += (size_t)blockIdx.y * T;

    const int q_lo = blockIdx.x * 4, q_hi = min(T - 1, q_lo + 3);
    const int q = q_lo + wave;
    const bool q_ok = q < T;
    const int qc = min(q, T - 1);
    const int a_lo = mask.causal ? max(0, q_lo - mask.wa) : 0, a_hi = mask.causal ? q_hi : T - 1;
    const int b_lo = mask.causal ? max(0, q_lo - mask.wb) : 0, b_hi = mask.causal ? q_hi : T - 1;

    float M = -INFINITY, L = 0.f, o0 = 0.f, o1 = 0.f;  // lane d holds O[d] (and O[d+64])
    for (int b0 = b_lo & ~63; b0 <= b_hi; b0 += 64) {
        const int b = b0 + lane, bc = min(b, T - 1);
        float qb[D], acc[D];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            qb[d] = Q[(size_t)qc * D + d] * KB[(size_t)bc * D + d] * scale_log2;
            acc[d] = 0.f;
        }
        float m = -INFINITY, l = 0.f;
        for (int a0 = a_lo & ~(kStageRows - 1); a0 <= a_hi; a0 += kStageRows) {
            __syncthreads();
            stage_rows<D>(sK, KA, a0, T);
            stage_rows<D>(sV, VA, a0, T);
            __syncthreads();
            const int n = min(kStageRows, a_hi - a0 + 1);
            for (int aa = 0; aa < n; ++aa) {
                const int a = a0 + aa;
                const float s = dot_lds<D>(qb, sK[aa]);
                const bool ok = q_ok && b < T && tdp_valid(mask, q, a, b);
                if (ok) {
                    if (s > m) {
                        const float f = fast_exp2(m - s);
                        l *= f;
#pragma unroll
                        for (int d = 0; d < D; ++d) acc[d] *= f;
                        m = s;
                    }
                    const float p = fast_exp2(s - m);
                    l += p;
                    axpy_lds<D>(acc, p, sV[aa]);
                }
            }
        }
        // merge the 64 rows (q, b) of this tile into the running (M, L, O) of query q
        const float m_tile = wave_max(m);
        if (m_tile > -INFINITY) {
            const float m_new = fmaxf(M, m_tile);
            const float f = fast_exp2(M - m_new);  // 0 when M = -inf
            const float w = (m > -INFINITY) ? fast_exp2(m - m_new) : 0.f;
            L = L * f + wave_sum(w * l);
            o0 *= f;
            o1 *= f;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const float t = wave_sum(w * acc[d] * VB[(size_t)bc * D + d]);
                if (d < 64) {
                    o0 = (lane == d) ? o0 + t : o0;
                } else {
                    o1 = (lane == d - 64) ? o1 + t : o1;
                }
            }
            M = m_new;
        }
    }
    if (q_ok) {
        const float inv = 1.0f / L;
        if (lane < D) O[(size_t)q * D + lane] = o0 * inv;
        if (D > 64 && lane + 64 < D) O[(size_t)q * D + lane + 64] = o1 * inv;
        if (lane == 0) LSE[q] = (M + fast_log2(L)) * kLn2;
    }
}

// ------------------------------------------------------------------------------------------
// Backward, owner = query.  Same decomposition as the forward; per lane (q, b):
//   P = exp2(s - lse2[q]),  dP = (dO[q]*VB[b]) . VA[a],  dS = P (dP - Delta[q]),
//   acc += dS * KA[a]   and after the sweep   dQ[q] += alpha * sum_b acc * KB[b].
template <int D>
__global__ __launch_bounds__(256) void tdp_bwd_q_generic_kernel(
    const float* __restrict__ Q, const float* __restrict__ KA, const float* __restrict__ KB,
    const float* __restrict__ VA, const float* __restrict__ VB, const float* __restrict__ dO,
    const float* __restrict__ LSE, const float* __restrict__ Delta, float* __restrict__ dQ, int T,
    float alpha, TdpMask mask) {
    __shared__ __align__(16) float sK[kStageRows][D];
    __shared__ __align__(16) float sV[kStageRows][D];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t base = (size_t)blockIdx.y * T * D;
    Q += base; KA += base; KB += base; VA += base; VB += base; dO += base; dQ += base;
    LSE += (size_t)blockIdx.y * T;
    Delta += (size_t)blockIdx.y * T;

    const int q_lo = blockIdx.x * 4, q_hi = min(T - 1, q_lo + 3);
    const int q = q_lo + wave;
    const bool q_ok = q < T;
    const int qc = min(q, T - 1);
    const int a_lo = mask.causal ? max(0, q_lo - mask.wa) : 0, a_hi = mask.causal ? q_hi : T - 1;
    const int b_lo = mask.causal ? max(0, q_lo - mask.wb) : 0, b_hi = mask.causal ? q_hi : T - 1;
    const float scale_log2 = alpha * kLog2e;
    const float lse2 = LSE[qc] * kLog2e, delta = Delta[qc];

    using RS = RowSplit<D>;
    constexpr int LP = RS::LP, DL = RS::DL, RPT = RS::RPT;
    const int lrow = lane % RPT, c0 = (lane / RPT) * DL;  // this lane's row of a tile and its first column

    float o0 = 0.f, o1 = 0.f;  // dQ[q][c0 + lrow] and dQ[q][c0 + lrow + RPT]
    for (int b0 = b_lo & ~(RPT - 1); b0 <= b_hi; b0 += RPT) {
        const int b = b0 + lrow, bc = min(b, T - 1);
        float qb[DL], gb[DL], acc[DL];
#pragma unroll
        for (int d = 0; d < DL; ++d) {
            const float kb = KB[(size_t)bc * D + c0 + d];
            qb[d] = Q[(size_t)qc * D + c0 + d] * kb * scale_log2;
            gb[d] = dO[(size_t)qc * D + c0 + d] * VB[(size_t)bc * D + c0 + d];
            acc[d] = 0.f;
        }
        for (int a0 = a_lo & ~(kStageRows - 1); a0 <= a_hi; a0 += kStageRows) {
            __syncthreads();
            stage_rows<D>(sK, KA, a0, T);
            stage_rows<D>(sV, VA, a0, T);
            __syncthreads();
            const int n = min(kStageRows, a_hi - a0 + 1);
            for (int aa = 0; aa < n; ++aa) {
                const int a = a0 + aa;
                const bool ok = q_ok && b < T && tdp_valid(mask, q, a, b);  // the same for the lanes of a row
                if (ok) {
                    const float s = join_parts<LP>(dot_lds<DL>(qb, sK[aa] + c0));
                    const float dp = join_parts<LP>(dot_lds<DL>(gb, sV[aa] + c0));
                    const float ds = fast_exp2(s - lse2) * (dp - delta);
                    axpy_lds<DL>(acc, ds, sK[aa] + c0);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < DL; ++d) {
            const float t = part_sum<LP>(acc[d] * KB[(size_t)bc * D + c0 + d]);
            if (d < RPT) {
                o0 = (lrow == d) ? o0 + t : o0;
            } else {
                o1 = (lrow == d - RPT) ? o1 + t : o1;
            }
        }
    }
    if (q_ok) {
        if (lrow < DL) dQ[(size_t)q * D + c0 + lrow] = o0 * alpha;
        if (DL > RPT) dQ[(size_t)q * D + c0 + lrow + RPT] = o1 * alpha;
    }
}

// ------------------------------------------------------------------------------------------
// Backward, owner = key row b (one per wave), lanes sweep the queries q in tiles of 64:
//   accK += dS * KA[a],  accV += P * VA[a]  over a;  then
//   dKB[b] += alpha * sum_q accK * Q[q],   dVB[b] += sum_q accV * dO[q].
// Called twice: (a,b) = (j,k) gives dK2, dV2; with the roles of (K1,U) and (K2,V2) exchanged
// (and the mask transposed) it gives dK1 and dU.
template <int D>
__global__ __launch_bounds__(256) void tdp_bwd_b_generic_kernel(
    const float* __restrict__ Q, const float* __restrict__ KA, const float* __restrict__ KB,
    const float* __restrict__ VA, const float* __restrict__ VB, const float* __restrict__ dO,
    const float* __restrict__ LSE, const float* __restrict__ Delta, float* __restrict__ dKB,
    float* __restrict__ dVB, int T, float alpha, TdpMask mask) {
    __shared__ __align__(16) float sK[kStageRows][D];
    __shared__ __align__(16) float sV[kStageRows][D];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t base = (size_t)blockIdx.y * T * D;
    Q += base; KA += base; KB += base; VA += base; VB += base; dO += base; dKB += base; dVB += base;
    LSE += (size_t)blockIdx.y * T;
    Delta += (size_t)blockIdx.y * T;

    const int b_lo = blockIdx.x * 4, b_hi = min(T - 1, b_lo + 3);
    const int b = b_lo + wave;
    const bool b_ok = b < T;
    const int bc = min(b, T - 1);
    const int q_lo = mask.causal ? b_lo : 0;
    const int q_hi = mask.causal ? min(T - 1, b_hi + mask.wb) : T - 1;
    const float scale_log2 = alpha * kLog2e;

    using RS = RowSplit<D>;
    constexpr int LP = RS::LP, DL = RS::DL, RPT = RS::RPT;
    const int lrow = lane % RPT, c0 = (lane / RPT) * DL;

    float k0 = 0.f, k1 = 0.f, v0 = 0.f, v1 = 0.f;  // columns c0 + lrow and c0 + lrow + RPT of dKB[b], dVB[b]
    for (int q0 = q_lo & ~(RPT - 1); q0 <= q_hi; q0 += RPT) {
        const int q = q0 + lrow, qc = min(q, T - 1);
        const int qt_hi = min(q_hi, q0 + RPT - 1);
        const int a_lo = mask.causal ? max(0, max(q0, q_lo) - mask.wa) : 0;
        const int a_hi = mask.causal ? qt_hi : T - 1;
        const float lse2 = LSE[qc] * kLog2e, delta = Delta[qc];
        float qb[DL], gb[DL], accK[DL], accV[DL];
#pragma unroll
        for (int d = 0; d < DL; ++d) {
            qb[d] = Q[(size_t)qc * D + c0 + d] * KB[(size_t)bc * D + c0 + d] * scale_log2;
            gb[d] = dO[(size_t)qc * D + c0 + d] * VB[(size_t)bc * D + c0 + d];
            accK[d] = 0.f;
            accV[d] = 0.f;
        }
        for (int a0 = a_lo & ~(kStageRows - 1); a0 <= a_hi; a0 += kStageRows) {
            __syncthreads();
            stage_rows<D>(sK, KA, a0, T);
            stage_rows<D>(sV, VA, a0, T);
            __syncthreads();
            const int n = min(kStageRows, a_hi - a0 + 1);
            for (int aa = 0; aa < n; ++aa) {
                const int a = a0 + aa;
                const bool ok = b_ok && q < T && q >= q_lo && tdp_valid(mask, q, a, b);  // the same for the lanes of a row
                if (ok) {
                    const float s = join_parts<LP>(dot_lds<DL>(qb, sK[aa] + c0));
                    const float dp = join_parts<LP>(dot_lds<DL>(gb, sV[aa] + c0));
                    const float p = fast_exp2(s - lse2);
                    axpy_lds<DL>(accK, p * (dp - delta), sK[aa] + c0);
                    axpy_lds<DL>(accV, p, sV[aa] + c0);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < DL; ++d) {
            const float tk = part_sum<LP>(accK[d] * Q[(size_t)qc * D + c0 + d]);
            const float tv = part_sum<LP>(accV[d] * dO[(size_t)qc * D + c0 + d]);
            if (d < RPT) {
                k0 = (lrow == d) ? k0 + tk : k0;
                v0 = (lrow == d) ? v0 + tv : v0;
            } else {
                k1 = (lrow == d - RPT) ? k1 + tk : k1;
                v1 = (lrow == d - RPT) ? v1 + tv : v1;
            }
        }
    }
    if (b_ok) {
        if (lrow < DL) {
            dKB[(size_t)b * D + c0 + lrow] = k0 * alpha;
            dVB[(size_t)b * D + c0 + lrow] = v0;
        }
        if (DL > RPT) {
            dKB[(size_t)b * D + c0 + lrow + RPT] = k1 * alpha;
            dVB[(size_t)b * D + c0 + lrow + RPT] = v1;
        }
    }
}

// ------------------------------------------------------------------------------------------
template <int D>
static hipError_t launch_fwd(const GenericTdpArgs& a, hipStream_t st) {
    dim3 grid((a.T + 3) / 4, a.BH);
    TdpMask m{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    hipLaunchKernelGGL(tdp_fwd_generic_kernel<D>, grid, dim3(256), 0, st, a.q, a.k1, a.k2, a.u, a.v2, a.o,
                       a.lse, a.T, a.alpha * kLog2e, m);
    return hipGetLastError();
}

template <int D>
static hipError_t launch_bwd(const GenericTdpArgs& a, hipStream_t st) {
    dim3 grid((a.T + 3) / 4, a.BH);
    TdpMask m{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    // transposed roles: staged = k (K2/V2), owner = j (K1/U)
    TdpMask mt{a.causal, a.k2_window, a.k1_window, a.kk_right, a.kk_left};
    // a null output pair is a launch the caller does not want
    if (a.dq)
        hipLaunchKernelGGL(tdp_bwd_q_generic_kernel<D>, grid, dim3(256), 0, st, a.q, a.k1, a.k2, a.u, a.v2,
                           a.d_o, a.lse_in, a.delta, a.dq, a.T, a.alpha, m);
    if (a.dk2 && a.dv2)
        hipLaunchKernelGGL(tdp_bwd_b_generic_kernel<D>, grid, dim3(256), 0, st, a.q, a.k1, a.k2, a.u, a.v2,
                           a.d_o, a.lse_in, a.delta, a.dk2, a.dv2, a.T, a.alpha, m);
    if (a.dk1 && a.du)
        hipLaunchKernelGGL(tdp_bwd_b_generic_kernel<D>, grid, dim3(256), 0, st, a.q, a.k2, a.k1, a.v2, a.u,
                           a.d_o, a.lse_in, a.delta, a.dk1, a.du, a.T, a.alpha, mt);
    return hipGetLastError();
}

hipError_t generic_tdp_fwd(const GenericTdpArgs& a, hipStream_t st) {
    switch (a.D) {
        case 8: return launch_fwd<8>(a, st);
        case 16: return launch_fwd<16>(a, st);
        case 32: return launch_fwd<32>(a, st);
        case 64: return launch_fwd<64>(a, st);
        case 128: return launch_fwd<128>(a, st);
    }
    return hipErrorInvalidValue;
}

hipError_t generic_tdp_bwd(const GenericTdpArgs& a, hipStream_t st) {
    switch (a.D) {
        case 8: return launch_bwd<8>(a, st);
        case 16: return launch_bwd<16>(a, st);
        case 32: return launch_bwd<32>(a, st);
        case 64: return launch_bwd<64>(a, st);
        case 128: return launch_bwd<128>(a, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace tritt
