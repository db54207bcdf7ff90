// Triple-dot-product trittention backward on MFMA (gfx950), 16-bit tensors, D = 64,
// full causal windows or no mask.
//
// With virtual query rows (q,k):  A = alpha*log2e * Q[q] (.) K2[k],  G = dO[q] (.) V2[k],
//   S = A K1^T (log2 units),  P = exp2(S - LSE2[q]),  dP = G U^T,  dS = P (dP - Delta[q])
// six contractions are needed per valid (q,j,k):
//   S, dP, dQK2 = dS K1, Tv = P U, dK1 += dS^T A, dU += P^T G
// They are evaluated by two kernels, each recomputing S and dP (8 products executed for 6):
//
//  * tdp_bwd_qk_kernel: owner = 8 queries (one per wave); same loop nest as the forward
//    (k-tiles of 32 outside, 64-row stages of K1/U inside).  Accumulates dQK2 and Tv over the
//    whole j loop in registers, then per k-tile:  dQ[q] += sum_k dQK2 (.) K2[k] (registers,
//    owner-computes), and the two per-k sums  dK2[k] += dQK2 (.) Q[q],  dV2[k] += Tv (.) dO[q]
//    are first reduced over the workgroup's 8 queries in LDS and then added to fp32 global
//    accumulators (one returnless atomic per element per (query group, k-tile)).
//
//  * tdp_bwd_j_kernel: owner = 256 K1/V1 rows (32 per wave, operands held in registers for the
//    whole kernel); streams virtual-row tiles (one q, 32 k) whose operands A, G and their
//    transposes are built cooperatively in LDS.  dK1/dU stay in registers; the query range is
//    split over NQC workgroups whose fp32 partial results are summed by the finishing kernel
//    (no atomics, fixed order).
#include <type_traits>

#include "kernels.hpp"
#include "mfma.hpp"

namespace tritt {

template <typename E>
struct BwdParams {
    const E *q, *k1, *k2, *v2, *d_o;
    const E *u, *ut, *k1t, *k2t, *v2t;  // scratch: SiLU(V1) [BH][T][D]; transposes [BH][D][Tp]
    const float *lse, *delta;  // [BH][T]
    E* dq;
    float *dk2acc, *dv2acc;    // [BH][T][D] fp32, zero on entry
    float *dk1part, *dupart;   // [NQC][BH][T][D] fp32
    int T, Tp, BH, nqt, nqc;
    float alpha;
    int causal;
};

// ------------------------------------------------------------------------------------------
template <typename E, int D>
__global__ __launch_bounds__(512) void tdp_bwd_qk_kernel(BwdParams<E> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = D / 32, BQ = 8;
    constexpr int LDK = D + 8, LDU = 64 + 8, LDA = D + 4;
    constexpr int CH = D / 64;

    extern __shared__ __align__(16) char smem[];
    E* sK1 = reinterpret_cast<E*>(smem);   // [2][64][LDK]
    E* sU = sK1 + 2 * 64 * LDK;            // [2][64][LDK]
    E* sK1T = sU + 2 * 64 * LDK;           // [2][D][LDU]
    E* sUT = sK1T + 2 * D * LDU;           // [2][D][LDU]
    E* sK2 = sUT + 2 * D * LDU;            // [2][32][LDK]
    E* sV2 = sK2 + 2 * 32 * LDK;           // [2][32][LDK]
    E* sQ = sV2 + 2 * 32 * LDK;            // [BQ][LDK]
    E* sDO = sQ + BQ * LDK;                // [BQ][LDK]
    float* sAccK = reinterpret_cast<float*>(sDO + BQ * LDK);  // [32][LDA]
    float* sAccV = sAccK + 32 * LDA;                          // [32][LDA]

    const int groups = (p.BH + 7) / 8;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int bh = (slot % groups) * 8 + xcd;
    const int qt = p.nqt - 1 - slot / groups;
    if (bh >= p.BH) return;

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * p.Tp;
    const E* __restrict__ K1 = p.k1 + base;
    const E* __restrict__ U = p.u + base;
    const E* __restrict__ K2 = p.k2 + base;
    const E* __restrict__ V2 = p.v2 + base;
    const E* __restrict__ K1T = p.k1t + tbase;
    const E* __restrict__ UT = p.ut + tbase;

    const int q0 = qt * BQ;
    const int jend = p.causal ? min(T - 1, q0 + BQ - 1) : T - 1;
    const int nst = jend / 64 + 1, nkt = jend / 32 + 1;
    const int q = q0 + wave;
    const bool q_ok = q < T;
    const int qc = min(q, T - 1);
    const int jmax = p.causal ? qc : T - 1;
    const float lse2 = p.lse[(size_t)bh * T + qc] * kLog2e;
    const float delta = p.delta[(size_t)bh * T + qc];
    const float scale_log2 = p.alpha * kLog2e;

    uint4 r1[CH], r2[CH], r3[CH], r4[CH], rkv[CH];
    auto issue_stage = [&](int st) {
        const int jb = st * 64;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int idx = tid + c * 512;
            const int r = idx / (D / 8), ch = idx % (D / 8);
            const size_t off = (size_t)min(jb + r, T - 1) * D + ch * 8;
            r1[c] = *reinterpret_cast<const uint4*>(K1 + off);
            r2[c] = *reinterpret_cast<const uint4*>(U + off);
            const int d = idx / 8, cj = idx % 8;
            const size_t offt = (size_t)d * p.Tp + jb + cj * 8;
            r3[c] = *reinterpret_cast<const uint4*>(K1T + offt);
            r4[c] = *reinterpret_cast<const uint4*>(UT + offt);
        }
    };
    auto commit_stage = [&](int buf) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int idx = tid + c * 512;
            const int r = idx / (D / 8), ch = idx % (D / 8);
            *reinterpret_cast<uint4*>(sK1 + (buf * 64 + r) * LDK + ch * 8) = r1[c];
            *reinterpret_cast<uint4*>(sU + (buf * 64 + r) * LDK + ch * 8) = r2[c];
            const int d = idx / 8, cj = idx % 8;
            *reinterpret_cast<uint4*>(sK1T + (buf * D + d) * LDU + cj * 8) = r3[c];
            *reinterpret_cast<uint4*>(sUT + (buf * D + d) * LDU + cj * 8) = r4[c];
        }
    };
    auto issue_ktile = [&](int kt) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int idx = tid + c * 512;
            const int which = idx / (4 * D), rem = idx % (4 * D);
            const int r = rem / (D / 8), ch = rem % (D / 8);
            const E* src = which ? V2 : K2;
            rkv[c] = *reinterpret_cast<const uint4*>(src + (size_t)min(kt * 32 + r, T - 1) * D + ch * 8);
        }
    };
    auto commit_ktile = [&](int buf) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int idx = tid + c * 512;
            const int which = idx / (4 * D), rem = idx % (4 * D);
            const int r = rem / (D / 8), ch = rem % (D / 8);
            E* dst = which ? sV2 : sK2;
            *reinterpret_cast<uint4*>(dst + (buf * 32 + r) * LDK + ch * 8) = rkv[c];
        }
    };

    // prologue: Q and dO rows of the group, zeroed LDS accumulators, first k-tile and stage
    for (int idx = tid; idx < 2 * BQ * (D / 8); idx += 512) {
        const int which = idx / (BQ * (D / 8)), rem = idx % (BQ * (D / 8));
        const int r = rem / (D / 8), ch = rem % (D / 8);
        const E* src = (which ? p.d_o : p.q) + base + (size_t)min(q0 + r, T - 1) * D + ch * 8;
        *reinterpret_cast<uint4*>((which ? sDO : sQ) + r * LDK + ch * 8) = *reinterpret_cast<const uint4*>(src);
    }
    for (int idx = tid; idx < 2 * 32 * LDA; idx += 512) sAccK[idx] = 0.f;  // sAccK and sAccV are adjacent
    issue_ktile(0);
    issue_stage(0);
    commit_ktile(0);
    commit_stage(0);
    __syncthreads();

    float dqpart[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) dqpart[dt] = 0.f;
    const int krow_off = key_of_row(n);
    const v8 ones = ones_operand<E>(g), off_lse = offset_operand<E>(lse2, g), off_delta = offset_operand<E>(delta, g);

    int gstage = 0;
    for (int kt = 0; kt < nkt; ++kt) {
        const int kb = kt & 1;
        if (kt + 1 < nkt) issue_ktile(kt + 1);

        v8 bq[KS], bg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int off = ks * 16 + g * 8;
            const v8 kv = *reinterpret_cast<const v8*>(sK2 + (kb * 32 + n) * LDK + off);
            const v8 vv = *reinterpret_cast<const v8*>(sV2 + (kb * 32 + n) * LDK + off);
            const v8 qv = *reinterpret_cast<const v8*>(sQ + wave * LDK + off);
            const v8 dv = *reinterpret_cast<const v8*>(sDO + wave * LDK + off);
            v8 a, b;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const v2 pa = M::pack((float)kv[e] * (float)qv[e] * scale_log2,
                                      (float)kv[e + 1] * (float)qv[e + 1] * scale_log2);
                const v2 pb = M::pack((float)vv[e] * (float)dv[e], (float)vv[e + 1] * (float)dv[e + 1]);
                a[e] = pa[0]; a[e + 1] = pa[1];
                b[e] = pb[0]; b[e + 1] = pb[1];
            }
            bq[ks] = a;
            bg[ks] = b;
        }

        f32x16 accQ[DT], accT[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                accQ[dt][i] = 0.f;
                accT[dt][i] = 0.f;
            }

        for (int st = 0; st < nst; ++st, ++gstage) {
            const int sb = gstage & 1;
            const bool more = (st + 1 < nst) || (kt + 1 < nkt);
            if (more) issue_stage(st + 1 < nst ? st + 1 : 0);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int jb = st * 64 + half * 32;
                if (jb > jmax) break;  // wave-uniform: nothing at or below the causal bound
                f32x16 s, dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                    dp[i] = 0.f;
                }
                const int rowoff = (sb * 64 + half * 32 + krow_off) * LDK + g * 8;
                // the extra k-step subtracts LSE2[q] from S and Delta[q] from dP inside the MFMA
                s = M::mma(ones, off_lse, s);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const v8 ka = *reinterpret_cast<const v8*>(sK1 + rowoff + ks * 16);
                    s = M::mma(ka, bq[ks], s);
                }
                dp = M::mma(ones, off_delta, dp);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const v8 ua = *reinterpret_cast<const v8*>(sU + rowoff + ks * 16);
                    dp = M::mma(ua, bg[ks], dp);
                }
                v8 pa[2], da[2];
                // P = exp2(S - LSE2), dS = P (dP - Delta), both packed as A operands of the next
                // products.  The masked variant is a separate (wave-uniform) branch so that interior
                // steps carry no predication at all.
                auto softmax_grad = [&](auto masked_tag) {
                    constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const int i = h * 8 + e;
                            float p0 = fast_exp2(s[i]), p1 = fast_exp2(s[i + 1]);
                            if constexpr (MASKED) {
                                p0 = (jb + key_of(g, i) <= jmax) ? p0 : 0.f;
                                p1 = (jb + key_of(g, i + 1) <= jmax) ? p1 : 0.f;
                            }
                            const v2 pp = M::pack(p0, p1);
                            const v2 dd = M::pack(p0 * dp[i], p1 * dp[i + 1]);
                            pa[h][e] = pp[0]; pa[h][e + 1] = pp[1];
                            da[h][e] = dd[0]; da[h][e + 1] = dd[1];
                        }
                    }
                };
                if (__builtin_amdgcn_readfirstlane(jb + 31 > jmax))
                    softmax_grad(std::true_type{});
                else
                    softmax_grad(std::false_type{});
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int toff = (sb * D + dt * 32 + n) * LDU + half * 32 + h * 16 + g * 8;
                        const v8 ub = *reinterpret_cast<const v8*>(sUT + toff);
                        const v8 kb1 = *reinterpret_cast<const v8*>(sK1T + toff);
                        accT[dt] = M::mma(pa[h], ub, accT[dt]);
                        accQ[dt] = M::mma(da[h], kb1, accQ[dt]);
                    }
                }
            }
            if (more) commit_stage(sb ^ 1);
            __syncthreads();
        }

        // ---- k-tile epilogue ------------------------------------------------------------------
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int d = dt * 32 + n;
            const float qd = (float)sQ[wave * LDK + d] * p.alpha;
            const float dod = (float)sDO[wave * LDK + d];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int r = c_row(g, i);
                const int k = kt * 32 + r;
                if (q_ok && k <= jmax) {
                    dqpart[dt] += accQ[dt][i] * (float)sK2[(kb * 32 + r) * LDK + d];
                    unsafeAtomicAdd(p.dk2acc + base + (size_t)k * D + d, accQ[dt][i] * qd);
                    unsafeAtomicAdd(p.dv2acc + base + (size_t)k * D + d, accT[dt][i] * dod);
                }
            }
        }
        if (kt + 1 < nkt) commit_ktile(kb ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const float v = (dqpart[dt] + __shfl_xor(dqpart[dt], 32, 64)) * p.alpha;
        if (q_ok && g == 0) p.dq[base + (size_t)q * D + dt * 32 + n] = (E)v;
    }
}

// ------------------------------------------------------------------------------------------
// Owner = 256 rows j of K1/V1 (32 per wave).  For one query q at a time ("round") the wave
// builds its B operands in registers
//   k1q[j, d] = alpha*log2e * Q[q,d] K1[j,d],   uq[j, d] = dO[q,d] U[j,d]
// and sweeps the k axis in stages of 64 rows shared by the whole workgroup:
//   S[k, j]  = K2[k,:] . k1q[j,:]        dP[k, j] = V2[k,:] . uq[j,:]
//   P = exp2(S - LSE2[q]),  dS = P (dP - Delta[q])
//   dK1[j, :] += dS^T (K2 (.) Q[q])      dU[j, :]  += P^T (V2 (.) dO[q])
// The two Hadamard-scaled transposed operands are written to LDS by the stage loader (from the
// pre-transposed K2^T / V2^T scratch, 8 keys per thread), so dK1/dU accumulate directly in
// registers over all rounds.  Workgroups split the queries NQC ways (round robin) and write fp32
// partial results that the finishing kernel adds in a fixed order.
template <typename E, int D>
__global__ __launch_bounds__(512) void tdp_bwd_j_kernel(BwdParams<E> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = D / 32, JB = 256;
    constexpr int LDK = D + 8, LDU = 64 + 8;
    static_assert(D == 64, "stage loader below assumes 512 threads x one 16-byte chunk per tensor");

    extern __shared__ __align__(16) char smem[];
    E* sK2 = reinterpret_cast<E*>(smem);   // [2][64][LDK]  rows k
    E* sV2 = sK2 + 2 * 64 * LDK;           // [2][64][LDK]
    E* sAT = sV2 + 2 * 64 * LDK;           // [2][D][LDU]   K2^T (.) Q[q]
    E* sGT = sAT + 2 * D * LDU;            // [2][D][LDU]   V2^T (.) dO[q]
    E* sQr = sGT + 2 * D * LDU;            // [2][D]  Q[q] of the round that starts in this buffer
    E* sOr = sQr + 2 * D;                  // [2][D]  dO[q]
    float* sMeta = reinterpret_cast<float*>(sOr + 2 * D);  // [2][2]  LSE2[q], Delta[q]

    const int njb = (p.T + JB - 1) / JB;
    int bid = blockIdx.x;
    // heaviest first: low j blocks see the most queries
    const int chunk = bid % p.nqc; bid /= p.nqc;
    const int bh = bid % p.BH;
    const int jb = bid / p.BH;
    (void)njb;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * p.Tp;
    const E* __restrict__ Q = p.q + base;
    const E* __restrict__ dO = p.d_o + base;
    const E* __restrict__ K2 = p.k2 + base;
    const E* __restrict__ V2 = p.v2 + base;
    const E* __restrict__ K2T = p.k2t + tbase;
    const E* __restrict__ V2T = p.v2t + tbase;
    const float* __restrict__ LSE = p.lse + (size_t)bh * T;
    const float* __restrict__ DEL = p.delta + (size_t)bh * T;
    const float scale_log2 = p.alpha * kLog2e;

    const int j0 = jb * JB, jw = j0 + wave * 32;
    const int jrow = min(jw + n, T - 1);
    v8 k1raw[KS], uraw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        k1raw[ks] = *reinterpret_cast<const v8*>(p.k1 + base + (size_t)jrow * D + ks * 16 + g * 8);
        uraw[ks] = *reinterpret_cast<const v8*>(p.u + base + (size_t)jrow * D + ks * 16 + g * 8);
    }
    f32x16 accK[DT], accU[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            accK[dt][i] = 0.f;
            accU[dt][i] = 0.f;
        }

    // rounds: q = q_first + chunk + nqc*m ; stages of round q: 0 .. kmax(q)/64
    const int q_first = p.causal ? j0 : 0;
    auto kmax_of = [&](int q) { return p.causal ? q : T - 1; };

    // stage loader: thread -> one 16-byte chunk of each of the four tensors
    const int lr = tid >> 3, lc = tid & 7;  // K2/V2: row lr, chunk lc ; K2T/V2T: d = lr, key chunk lc
    uint4 l1, l2, l3, l4;
    E lqd, lod;
    auto issue_stage = [&](int q, int st) {
        const int kb = st * 64;
        const size_t off = (size_t)min(kb + lr, T - 1) * D + lc * 8;
        l1 = *reinterpret_cast<const uint4*>(K2 + off);
        l2 = *reinterpret_cast<const uint4*>(V2 + off);
        const size_t offt = (size_t)lr * p.Tp + kb + lc * 8;
        l3 = *reinterpret_cast<const uint4*>(K2T + offt);
        l4 = *reinterpret_cast<const uint4*>(V2T + offt);
        lqd = Q[(size_t)q * D + lr];
        lod = dO[(size_t)q * D + lr];
    };
    auto commit_stage = [&](int buf, int q, int st) {
        *reinterpret_cast<uint4*>(sK2 + (buf * 64 + lr) * LDK + lc * 8) = l1;
        *reinterpret_cast<uint4*>(sV2 + (buf * 64 + lr) * LDK + lc * 8) = l2;
        const v8 kt = *reinterpret_cast<const v8*>(&l3), vt = *reinterpret_cast<const v8*>(&l4);
        const float qd = (float)lqd, od = (float)lod;
        v8 a, gg;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const v2 pa = M::pack((float)kt[e] * qd, (float)kt[e + 1] * qd);
            const v2 pb = M::pack((float)vt[e] * od, (float)vt[e + 1] * od);
            a[e] = pa[0]; a[e + 1] = pa[1];
            gg[e] = pb[0]; gg[e + 1] = pb[1];
        }
        *reinterpret_cast<v8*>(sAT + (buf * D + lr) * LDU + lc * 8) = a;
        *reinterpret_cast<v8*>(sGT + (buf * D + lr) * LDU + lc * 8) = gg;
        if (st == 0) {  // first stage of a round also carries the round's query row and scalars
            if (lc == 0) {
                sQr[buf * D + lr] = lqd;
                sOr[buf * D + lr] = lod;
            }
            if (tid == 0) {
                sMeta[buf * 2] = LSE[q] * kLog2e;
                sMeta[buf * 2 + 1] = DEL[q];
            }
        }
    };

    int cq = q_first + chunk, cst = 0;  // current (round, stage)
    bool have = cq < T;
    if (have) {
        issue_stage(cq, 0);
        commit_stage(0, cq, 0);
    }
    __syncthreads();

    const int krow_off = key_of_row(n);
    v8 k1q[KS], uq[KS];
    const v8 ones = ones_operand<E>(g);
    v8 off_lse = ones, off_delta = ones;
    int buf = 0;
    while (have) {
        const int kmax = kmax_of(cq), jlim = p.causal ? cq : T - 1;
        const bool active = (jw <= jlim) && (jw < T);  // wave-uniform
        int nq = cq, nst = cst + 1;
        if (nst * 64 > kmax) {
            nq = cq + p.nqc;
            nst = 0;
        }
        const bool next = nq < T;
        if (next) issue_stage(nq, nst);

        if (cst == 0 && active) {
            // new round: operands of this wave for query cq
            off_lse = offset_operand<E>(sMeta[buf * 2], g);
            off_delta = offset_operand<E>(sMeta[buf * 2 + 1], g);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v8 qv = *reinterpret_cast<const v8*>(sQr + buf * D + ks * 16 + g * 8);
                const v8 ov = *reinterpret_cast<const v8*>(sOr + buf * D + ks * 16 + g * 8);
                v8 a, b;
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const v2 pa = M::pack((float)k1raw[ks][e] * (float)qv[e] * scale_log2,
                                          (float)k1raw[ks][e + 1] * (float)qv[e + 1] * scale_log2);
                    const v2 pb = M::pack((float)uraw[ks][e] * (float)ov[e], (float)uraw[ks][e + 1] * (float)ov[e + 1]);
                    a[e] = pa[0]; a[e + 1] = pa[1];
                    b[e] = pb[0]; b[e + 1] = pb[1];
                }
                k1q[ks] = a;
                uq[ks] = b;
            }
        }

        if (active) {
            const bool jok = (jw + n <= jlim) && (jw + n < T);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int kb = cst * 64 + half * 32;
                if (kb > kmax) break;
                f32x16 s, dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                    dp[i] = 0.f;
                }
                const int rowoff = (buf * 64 + half * 32 + krow_off) * LDK + g * 8;
                s = M::mma(ones, off_lse, s);  // S - LSE2[q], dP - Delta[q] come out of the MFMA
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    s = M::mma(*reinterpret_cast<const v8*>(sK2 + rowoff + ks * 16), k1q[ks], s);
                dp = M::mma(ones, off_delta, dp);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    dp = M::mma(*reinterpret_cast<const v8*>(sV2 + rowoff + ks * 16), uq[ks], dp);
                const bool diag = (kb + 31 > kmax) || (jw + 31 > jlim) || (jw + 31 >= T);
                v8 pa[2], da[2];
                auto softmax_grad = [&](auto masked_tag) {
                    constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const int i = h * 8 + e;
                            float p0 = fast_exp2(s[i]), p1 = fast_exp2(s[i + 1]);
                            if constexpr (MASKED) {
                                p0 = (jok && kb + key_of(g, i) <= kmax) ? p0 : 0.f;
                                p1 = (jok && kb + key_of(g, i + 1) <= kmax) ? p1 : 0.f;
                            }
                            const v2 pp = M::pack(p0, p1);
                            const v2 dd = M::pack(p0 * dp[i], p1 * dp[i + 1]);
                            pa[h][e] = pp[0]; pa[h][e + 1] = pp[1];
                            da[h][e] = dd[0]; da[h][e + 1] = dd[1];
                        }
                    }
                };
                if (__builtin_amdgcn_readfirstlane(diag))
                    softmax_grad(std::true_type{});
                else
                    softmax_grad(std::false_type{});
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int toff = (buf * D + dt * 32 + n) * LDU + half * 32 + h * 16 + g * 8;
                        accK[dt] = M::mma(da[h], *reinterpret_cast<const v8*>(sAT + toff), accK[dt]);
                        accU[dt] = M::mma(pa[h], *reinterpret_cast<const v8*>(sGT + toff), accU[dt]);
                    }
                }
            }
        }
        if (next) commit_stage(buf ^ 1, nq, nst);
        __syncthreads();
        buf ^= 1;
        cq = nq;
        cst = nst;
        have = next;
    }

    // partial results of this query chunk (dK1 still lacks the factor alpha: applied by the finisher)
    float* outK = p.dk1part + ((size_t)chunk * p.BH + bh) * T * D;
    float* outU = p.dupart + ((size_t)chunk * p.BH + bh) * T * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int j = jw + c_row(g, i);
            if (j < T) {
                outK[(size_t)j * D + dt * 32 + n] = accK[dt][i];
                outU[(size_t)j * D + dt * 32 + n] = accU[dt][i];
            }
        }
}

// ------------------------------------------------------------------------------------------
// scratch producers / consumers
// U = SiLU(V1) row-major; U^T and K1^T as [D][Tp] (zero padded); Delta = rowsum(dO*O);
// zero the fp32 accumulators.
template <typename E>
__global__ __launch_bounds__(256) void bwd_prep_kernel(const E* __restrict__ v1, const E* __restrict__ k1,
                                                       const E* __restrict__ k2, const E* __restrict__ v2,
                                                       const E* __restrict__ o, const E* __restrict__ d_o,
                                                       E* __restrict__ u, E* __restrict__ ut, E* __restrict__ k1t,
                                                       E* __restrict__ k2t, E* __restrict__ v2t,
                                                       float* __restrict__ delta, float* __restrict__ zero_a,
                                                       float* __restrict__ zero_b, int T, int Tp, int D) {
    const int bh = blockIdx.y, j0 = blockIdx.x * 64;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * Tp;
    for (int idx = threadIdx.x; idx < D * 64; idx += 256) {
        const int d = idx >> 6, jj = idx & 63, j = j0 + jj;
        float uv = 0.f, kv = 0.f, k2v = 0.f, v2v = 0.f;
        if (j < T) {
            const size_t off = base + (size_t)j * D + d;
            uv = silu_f((float)v1[off]);
            kv = (float)k1[off];
            k2v = (float)k2[off];
            v2v = (float)v2[off];
        }
        ut[tbase + (size_t)d * Tp + j] = (E)uv;
        k1t[tbase + (size_t)d * Tp + j] = (E)kv;
        k2t[tbase + (size_t)d * Tp + j] = (E)k2v;
        v2t[tbase + (size_t)d * Tp + j] = (E)v2v;
    }
    for (int idx = threadIdx.x; idx < D * 64; idx += 256) {
        const int jj = idx / D, d = idx % D, j = j0 + jj;
        if (j < T) {
            const size_t off = base + (size_t)j * D + d;
            u[off] = (E)silu_f((float)v1[off]);
            zero_a[off] = 0.f;
            zero_b[off] = 0.f;
        }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int jj = wave; jj < 64; jj += 4) {
        const int j = j0 + jj;
        if (j >= T) break;
        float part = 0.f;
        for (int d = lane; d < D; d += 64)
            part += (float)o[base + (size_t)j * D + d] * (float)d_o[base + (size_t)j * D + d];
        part = wave_sum(part);
        if (lane == 0) delta[(size_t)bh * T + j] = part;
    }
}

// dK1 = alpha * sum_c part_c ; dV1 = SiLU'(V1) * sum_c part_c ; dK2, dV2 = converted accumulators
template <typename E>
__global__ __launch_bounds__(256) void bwd_finish_kernel(const float* __restrict__ dk1part,
                                                         const float* __restrict__ dupart,
                                                         const float* __restrict__ dk2acc,
                                                         const float* __restrict__ dv2acc, const E* __restrict__ v1,
                                                         E* __restrict__ dk1, E* __restrict__ dv1, E* __restrict__ dk2,
                                                         E* __restrict__ dv2, size_t n, int nqc, float alpha) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float a = 0.f, b = 0.f;
        for (int c = 0; c < nqc; ++c) {
            a += dk1part[(size_t)c * n + i];
            b += dupart[(size_t)c * n + i];
        }
        dk1[i] = (E)(a * alpha);
        dv1[i] = (E)(b * silu_grad_f((float)v1[i]));
        dk2[i] = (E)dk2acc[i];
        dv2[i] = (E)dv2acc[i];
    }
}

constexpr int kNqc = 8;

struct BwdLayout {
    size_t u, ut, k1t, k2t, v2t, delta, dk2acc, dv2acc, dk1part, dupart, total;
};
static BwdLayout bwd_layout(int BH, int T, int D) {
    const size_t Tp = (size_t)(T + 63) / 64 * 64, n = (size_t)BH * T * D;
    BwdLayout l{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        off = (off + 255) & ~size_t(255);
        size_t r = off;
        off += bytes;
        return r;
    };
    l.u = take(n * 2);
    l.ut = take((size_t)BH * D * Tp * 2);
    l.k1t = take((size_t)BH * D * Tp * 2);
    l.k2t = take((size_t)BH * D * Tp * 2);
    l.v2t = take((size_t)BH * D * Tp * 2);
    l.delta = take((size_t)BH * T * 4);
    l.dk2acc = take(n * 4);
    l.dv2acc = take(n * 4);
    l.dk1part = take(n * 4 * kNqc);
    l.dupart = take(n * 4 * kNqc);
    l.total = (off + 255) & ~size_t(255);
    return l;
}

template <typename E, int D>
static hipError_t launch_bwd(const MfmaBwdArgs& a, hipStream_t st) {
    const int Tp = (a.T + 63) / 64 * 64;
    const BwdLayout l = bwd_layout(a.BH, a.T, D);
    char* ws = static_cast<char*>(a.workspace);
    BwdParams<E> p;
    p.q = (const E*)a.q; p.k1 = (const E*)a.k1; p.k2 = (const E*)a.k2; p.v2 = (const E*)a.v2;
    p.d_o = (const E*)a.d_o;
    p.u = (const E*)(ws + l.u); p.ut = (const E*)(ws + l.ut); p.k1t = (const E*)(ws + l.k1t);
    p.k2t = (const E*)(ws + l.k2t); p.v2t = (const E*)(ws + l.v2t);
    p.lse = a.lse; p.delta = (const float*)(ws + l.delta);
    p.dq = (E*)a.dq;
    p.dk2acc = (float*)(ws + l.dk2acc); p.dv2acc = (float*)(ws + l.dv2acc);
    p.dk1part = (float*)(ws + l.dk1part); p.dupart = (float*)(ws + l.dupart);
    p.T = a.T; p.Tp = Tp; p.BH = a.BH; p.nqt = (a.T + 7) / 8; p.nqc = kNqc;
    p.alpha = a.alpha; p.causal = a.causal;

    hipLaunchKernelGGL(bwd_prep_kernel<E>, dim3(Tp / 64, a.BH), dim3(256), 0, st, (const E*)a.v1, (const E*)a.k1,
                       (const E*)a.k2, (const E*)a.v2, (const E*)a.o, (const E*)a.d_o, (E*)(ws + l.u),
                       (E*)(ws + l.ut), (E*)(ws + l.k1t), (E*)(ws + l.k2t), (E*)(ws + l.v2t),
                       (float*)(ws + l.delta), p.dk2acc, p.dv2acc, a.T, Tp, D);

    constexpr size_t smem = 2 * (size_t)(2 * 2 * 64 * (D + 8) + 2 * 2 * D * 72 + 2 * 2 * 32 * (D + 8) + 2 * 8 * (D + 8)) +
                            2 * 32 * (D + 4) * 4;
    auto kern = tdp_bwd_qk_kernel<E, D>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int groups = (a.BH + 7) / 8;
    hipLaunchKernelGGL(kern, dim3(8 * groups * p.nqt), dim3(512), smem, st, p);

    const int njb = (a.T + 255) / 256;
    constexpr size_t smem_j = 2 * (size_t)(2 * 2 * 64 * (D + 8) + 2 * 2 * D * 72 + 2 * 2 * D) + 16;
    auto kern_j = tdp_bwd_j_kernel<E, D>;
    static bool attr_j = false;
    if (!attr_j) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern_j),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_j);
        if (e != hipSuccess) return e;
        attr_j = true;
    }
    hipLaunchKernelGGL(kern_j, dim3(a.BH * njb * kNqc), dim3(512), smem_j, st, p);

    const size_t n = (size_t)a.BH * a.T * D;
    size_t gridf = (n + 255) / 256;
    if (gridf > 4096) gridf = 4096;
    hipLaunchKernelGGL(bwd_finish_kernel<E>, dim3((unsigned)gridf), dim3(256), 0, st, (const float*)p.dk1part,
                       (const float*)p.dupart, (const float*)p.dk2acc, (const float*)p.dv2acc, (const E*)a.v1,
                       (E*)a.dk1, (E*)a.dv1, (E*)a.dk2, (E*)a.dv2, n, kNqc, a.alpha);
    return hipGetLastError();
}

size_t mfma_tdp_bwd_workspace(int BH, int T, int D) { return bwd_layout(BH, T, D).total; }
bool mfma_tdp_bwd_supported(int D, int dtype_is_16bit) { return dtype_is_16bit && D == 64; }

hipError_t mfma_tdp_bwd(const MfmaBwdArgs& a, hipStream_t st) {
    if (a.D != 64) return hipErrorInvalidValue;
    return a.is_bf16 ? launch_bwd<__bf16, 64>(a, st) : launch_bwd<_Float16, 64>(a, st);
}

}  // namespace tritt
