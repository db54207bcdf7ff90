// Triple-dot-product trittention backward on MFMA (gfx950), 16-bit tensors, D = 64,
// full causal windows or no mask.
//
// With virtual query rows (q,k):  A = alpha*log2e * Q[q] (.) K2[k],  G = dO[q] (.) V2[k],
//   S = A K1^T (log2 units),  P = exp2(S - LSE2[q]),  dP = G U^T,  dS = P (dP - Delta[q])
// six contractions are needed per valid (q,j,k):
//   S, dP, dQK2 = dS K1, Tv = P U, dK1 += dS^T A, dU += P^T G
// They are evaluated by two kernels, each recomputing S and dP (8 products executed for 6):
//
//  * tdp_bwd_qk_kernel: owner = 32 queries; tiles are (32 q) x (1 k), j is streamed.  Produces dQ
//    (owner-computes) and dK2 / dV2 (one fp32 atomic per element per (query tile, k)).
//  * tdp_bwd_j_kernel: owner = 256 K1/V1 rows; per query, k is streamed.  Produces dK1 / dV1 with
//    no atomics (fp32 partials per query chunk, summed in a fixed order by the finishing kernel).
// See the comment above each kernel.
#include <type_traits>

#include "direct_lds.hpp"
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
// Owner = 32 consecutive queries (the columns of every MFMA tile of the workgroup).  The eight
// waves take eight consecutive K2/V2 rows k per "round" (one k per wave), so a tile is
// (32 q) x (1 k), and sweep j in 64-row stages of K1 / U (and their transposes) shared by the
// workgroup.  Per round and wave, over the whole j sweep:
//   Yq[(q,k), :] = sum_j dS K1[j, :]        Tv[(q,k), :] = sum_j P U[j, :]
// and then
//   dQ[q]  += Yq (.) K2[k]                      (registers, all rounds; reduced over waves at the end)
//   dK2[k] += alpha * sum_q Yq (.) Q[q]         (sum over the tile's 32 rows in registers, then ONE
//   dV2[k] += sum_q Tv (.) dO[q]                 returnless fp32 atomic per element per (q-tile, k))
template <typename E, int D>
__global__ __launch_bounds__(512) void tdp_bwd_qk_kernel(BwdParams<E> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = D / 32, BQ = 32;
    constexpr int LDK = D + 8, LDF = D + 4;
    constexpr int TILE = 64 * 64;  // elements of one dense, swizzled 64x64 stage tile (see direct_lds.hpp)
    constexpr int NBUF = 3, LW = 4;  // stages in flight; direct loads per wave per stage
    static_assert(D == 64, "stages are four 64x64 tiles = 32 blocks of 1 KB, four per wave");

    extern __shared__ __align__(16) char smem[];
    E* sStage = reinterpret_cast<E*>(smem);  // [NBUF][4 tensors: K1, U, K1^T, U^T][TILE]
    E* sKr = sStage + NBUF * 4 * TILE;       // [2][8][D]  K2 rows of a round (one per wave), dense
    E* sVr = sKr + 2 * 8 * D;                // [2][8][D]  V2 rows
    E* sQb = sVr + 2 * 8 * D;                // [BQ][LDK]  Q tile (operand build)
    E* sOb = sQb + BQ * LDK;               // [BQ][LDK]    dO tile
    float* sQf = reinterpret_cast<float*>(sOb + BQ * LDK);  // [BQ][LDF]  alpha * Q, fp32 (epilogue)
    float* sOf = sQf + BQ * LDF;                            // [BQ][LDF]  dO, fp32

    const int groups = (p.BH + 7) / 8;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int bh = (slot % groups) * 8 + xcd;
    const int qt = p.nqt - 1 - slot / groups;  // heaviest query tiles first
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
    const int qlast = min(T - 1, q0 + BQ - 1);
    const int jend = p.causal ? qlast : T - 1;  // last j (and last k) any query of the tile needs
    const int nst = jend / 64 + 1, nrounds = jend / 8 + 1;
    const int q = q0 + n;                        // this lane's column
    const bool q_ok = q < T;
    const int jq = p.causal ? min(q, T - 1) : T - 1;  // per-lane bound on j and k
    const float scale_log2 = p.alpha * kLog2e;

    // stage loader: wave w fetches blocks 4*(w%2) .. +3 (8 rows each) of tensor w/2, direct to LDS
    const int tensor = wave >> 1;
    const bool rowmajor = tensor < 2;  // K1 / U: row = key j (read with permuted rows); else row = d
    const E* gsrc = uniform_ptr(tensor == 0 ? K1 : tensor == 1 ? U : tensor == 2 ? K1T : UT);
    auto issue_stage = [&](int st, int buf) {
        const int jb = st * 64;
        int ln = lane;
        asm volatile("" : "+v"(ln));  // keep this address arithmetic inside the loops (no spilled invariants)
        const int pos = ln & 7, rr = ln >> 3;
        E* dst = sStage + (buf * 4 + tensor) * TILE;
#pragma unroll
        for (int c = 0; c < LW; ++c) {
            const int blk = (wave & 1) * 4 + c, r = blk * 8 + rr;
            const unsigned off = rowmajor ? (unsigned)min(jb + r, T - 1) * (D * 2) + ((pos ^ swz_perm(r)) * 16)
                                          : ((unsigned)r * p.Tp + jb) * 2 + ((pos ^ swz_seq(r)) * 16);
            direct_load_16(gsrc, off, dst + blk * 512);
        }
    };
    auto issue_round = [&](int m, int buf) {  // waves 0, 1: K2 / V2 rows 8m .. 8m+7 (1 KB each)
        if (wave < 2) {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const unsigned off = (unsigned)min(m * 8 + (ln >> 3), T - 1) * (D * 2) + (ln & 7) * 16;
            direct_load_16(uniform_ptr(wave ? V2 : K2), off, (wave ? sVr : sKr) + buf * 8 * D);
        }
    };

    // prologue: Q / dO tiles in both forms, first round, first stage
    for (int idx = tid; idx < BQ * D; idx += 512) {
        const int r = idx / D, d = idx % D;
        const size_t off = base + (size_t)min(q0 + r, T - 1) * D + d;
        const E qv = p.q[off], ov = p.d_o[off];
        sQb[r * LDK + d] = qv;
        sOb[r * LDK + d] = ov;
        sQf[r * LDF + d] = (float)qv * p.alpha;
        sOf[r * LDF + d] = (float)ov;
    }
    issue_stage(0, 0);
    issue_stage(nst > 1 ? 1 : 0, 1);
    issue_round(0, 0);
    wait_vmcnt<0>();
    __syncthreads();

    // per-column constants folded into the score products (see offset_operand); a column past the
    // end of the sequence gets a huge LSE so that its P underflows to exactly 0
    const float lse2 = q_ok ? p.lse[(size_t)bh * T + q] * kLog2e : 3.0e4f;  // representable in fp16 too
    const float delta = q_ok ? p.delta[(size_t)bh * T + q] : 0.f;
    const v8 ones = ones_operand<E>(g), off_lse = offset_operand<E>(lse2, g), off_delta = offset_operand<E>(delta, g);
    const int krow_off = key_of_row(n);
    const int fperm = swz_perm(krow_off), fseq = swz_seq(n);

    f32x16 dQacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) dQacc[dt][i] = 0.f;

    int gstage = 0;
    for (int m = 0; m < nrounds; ++m) {
        const int mb = m & 1;
        const int k = m * 8 + wave;                 // this wave's K2/V2 row
        const bool k_active = k <= jend;            // wave-uniform
        const bool k_diag = p.causal && k > q0;     // some columns of the tile have q < k
        const bool kv_ok = !p.causal || k <= jq;    // per lane

        v8 bq[KS], bg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int off = ks * 16 + g * 8;
            const v8 kv = *reinterpret_cast<const v8*>(sKr + (mb * 8 + wave) * D + off);
            const v8 vv = *reinterpret_cast<const v8*>(sVr + (mb * 8 + wave) * D + off);
            const v8 qv = *reinterpret_cast<const v8*>(sQb + n * LDK + off);
            const v8 dv = *reinterpret_cast<const v8*>(sOb + n * LDK + off);
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
            const int sb = gstage % NBUF;
            // this stage has landed for every wave and the buffer two stages ahead is free; the j
            // sweep repeats every round, so the stages fetched ahead simply cycle
            barrier_keep_loads<LW>();
            if (st == 0 && m + 1 < nrounds) issue_round(m + 1, mb ^ 1);  // older than the stage loads below
            int st2 = st + 2;
            if (st2 >= nst) st2 -= nst;
            if (st2 >= nst) st2 = 0;
            issue_stage(st2, (gstage + 2) % NBUF);
            const E* sK1 = sStage + (sb * 4 + 0) * TILE;
            const E* sU = sStage + (sb * 4 + 1) * TILE;
            const E* sK1T = sStage + (sb * 4 + 2) * TILE;
            const E* sUT = sStage + (sb * 4 + 3) * TILE;
            if (k_active) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int jb = st * 64 + half * 32;
                    if (jb > jend) break;
                    f32x16 s, dp;
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        s[i] = 0.f;
                        dp[i] = 0.f;
                    }
                    const int rowoff = (half * 32 + krow_off) * 64;
                    // the extra k-step subtracts LSE2[q] from S and Delta[q] from dP inside the MFMA
                    s = M::mma(ones, off_lse, s);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        s = M::mma(*reinterpret_cast<const v8*>(sK1 + rowoff + (((ks * 2 + g) ^ fperm) * 8)), bq[ks], s);
                    dp = M::mma(ones, off_delta, dp);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        dp = M::mma(*reinterpret_cast<const v8*>(sU + rowoff + (((ks * 2 + g) ^ fperm) * 8)), bg[ks], dp);
                    v8 pa[2], da[2];
                    // P = exp2(S - LSE2), dS = P (dP - Delta), packed as A operands of the next products.
                    // The masked variant is a separate (wave-uniform) branch: interior steps carry no
                    // predication.
                    auto softmax_grad = [&](auto masked_tag) {
                        constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
#pragma unroll
                            for (int e = 0; e < 8; e += 2) {
                                const int i = h * 8 + e;
                                float p0 = fast_exp2(s[i]), p1 = fast_exp2(s[i + 1]);
                                if constexpr (MASKED) {
                                    p0 = (kv_ok && jb + key_of(g, i) <= jq) ? p0 : 0.f;
                                    p1 = (kv_ok && jb + key_of(g, i + 1) <= jq) ? p1 : 0.f;
                                }
                                const v2 pp = M::pack(p0, p1);
                                const v2 dd = M::pack(p0 * dp[i], p1 * dp[i + 1]);
                                pa[h][e] = pp[0]; pa[h][e + 1] = pp[1];
                                da[h][e] = dd[0]; da[h][e + 1] = dd[1];
                            }
                        }
                    };
                    if (__builtin_amdgcn_readfirstlane(k_diag || (p.causal && jb + 31 > q0) || jb + 31 > T - 1))
                        softmax_grad(std::true_type{});
                    else
                        softmax_grad(std::false_type{});
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int toff = (dt * 32 + n) * 64 + (((half * 4 + h * 2 + g) ^ fseq) * 8);
                            accT[dt] = M::mma(pa[h], *reinterpret_cast<const v8*>(sUT + toff), accT[dt]);
                            accQ[dt] = M::mma(da[h], *reinterpret_cast<const v8*>(sK1T + toff), accQ[dt]);
                        }
                    }
                }
            }
        }

        // ---- round epilogue (rows of the accumulators = the 32 queries, column = d) ---------------
        if (k_active) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 32 + n;
                const float kd = (float)sKr[(mb * 8 + wave) * D + d];
                float sk = 0.f, sv = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int r = c_row(g, i);
                    dQacc[dt][i] += accQ[dt][i] * kd;
                    sk += accQ[dt][i] * sQf[r * LDF + d];
                    sv += accT[dt][i] * sOf[r * LDF + d];
                }
                sk += __shfl_xor(sk, 32, 64);
                sv += __shfl_xor(sv, 32, 64);
                if (g == 0) {
                    unsafeAtomicAdd(p.dk2acc + base + (size_t)k * D + d, sk);
                    unsafeAtomicAdd(p.dv2acc + base + (size_t)k * D + d, sv);
                }
            }
        }
        // all waves are done with this round's K2/V2 rows and with the last stage
        barrier_keep_loads<LW>();
    }
    wait_vmcnt<0>();  // the stages fetched ahead land in the buffers reused below
    __syncthreads();

    // ---- dQ: sum the eight waves' partial tiles through LDS (the stage buffers are free now) ------
    float* red = reinterpret_cast<float*>(smem);  // [8][32][LDF]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) red[(wave * 32 + c_row(g, i)) * LDF + dt * 32 + n] = dQacc[dt][i];
    __syncthreads();
    for (int idx = tid; idx < BQ * D; idx += 512) {
        const int r = idx / D, d = idx % D;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) v += red[(w * 32 + r) * LDF + d];
        if (q0 + r < T) p.dq[base + (size_t)(q0 + r) * D + d] = (E)(v * p.alpha);
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

    // XCD-aware, heaviest-first block order: consecutive block ids go to different XCDs, so each
    // XCD keeps its own heads (their K2/V2 streams stay in that XCD's L2); low j blocks (which see
    // the most queries) are handed out first
    const int groups = (p.BH + 7) / 8;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int bh = (slot % groups) * 8 + xcd;
    const int rest = slot / groups;
    const int chunk = rest % p.nqc, jb = rest / p.nqc;
    if (bh >= p.BH) return;
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
    p.T = a.T; p.Tp = Tp; p.BH = a.BH; p.nqt = (a.T + 31) / 32; p.nqc = kNqc;
    p.alpha = a.alpha; p.causal = a.causal;

    hipLaunchKernelGGL(bwd_prep_kernel<E>, dim3(Tp / 64, a.BH), dim3(256), 0, st, (const E*)a.v1, (const E*)a.k1,
                       (const E*)a.k2, (const E*)a.v2, (const E*)a.o, (const E*)a.d_o, (E*)(ws + l.u),
                       (E*)(ws + l.ut), (E*)(ws + l.k1t), (E*)(ws + l.k2t), (E*)(ws + l.v2t),
                       (float*)(ws + l.delta), p.dk2acc, p.dv2acc, a.T, Tp, D);

    constexpr size_t smem = 2 * (size_t)(3 * 4 * 64 * 64 + 2 * 2 * 8 * D + 2 * 32 * (D + 8)) + 4 * (size_t)(2 * 32 * (D + 4));
    static_assert(smem >= 4 * 8 * 32 * (D + 4), "dQ reduction reuses the stage buffers");
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
    hipLaunchKernelGGL(kern_j, dim3(8 * groups * njb * kNqc), dim3(512), smem_j, st, p);

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
