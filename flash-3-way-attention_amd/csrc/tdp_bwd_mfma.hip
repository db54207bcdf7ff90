// Triple-dot-product trittention backward on MFMA (gfx950), 16-bit tensors.  This file: the kernel
// for D = 64 with full causal windows or no mask, the scratch producers / consumers and the launcher;
// tdp_bwd_rows_general.hpp: D = 128 and windowed masks.
//
// With virtual query rows (q,k):  A = alpha*log2e * Q[q] (.) K2[k],  G = dO[q] (.) V2[k],
//   S = A K1^T (log2 units),  P = exp2(S - LSE2[q]),  dP = G U^T,  dS = P (dP - Delta[q])
// six contractions are needed per valid (q,j,k):
//   S, dP, dS K1 (-> dQ, dK2), P U (-> dV2), and by the symmetry (K1,U,j) <-> (K2,V2,k) of the
//   whole problem, dS K2 (-> dK1) and P V2 (-> dU).
// One kernel template, tdp_bwd_rows_kernel, is launched twice, each launch recomputing S and dP
// (8 products executed for 6):
//   launch 1: rows = (K2, V2), streamed = (K1, U):  dQ (owner-computes), dK2, dV2
//   launch 2: rows = (K1, U),  streamed = (K2, V2): dK1, dU
// See the comment above the kernel.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "direct_lds.hpp"
#include "kernels.hpp"
#include "mfma.hpp"

namespace tritt {

__device__ __forceinline__ int wave_of(unsigned tid) { return __builtin_amdgcn_readfirstlane(tid >> 6); }

template <typename E>
struct BwdParams {
    const E *q, *d_o;
    // SV ("strided views") instantiations only: layouts of q, d_o, row_k, row_v, st_k, st_v (the caller's strides for
    // the caller's tensors, dense ones for SiLU(V1), which the workspace holds) and heads per batch entry; the other
    // instantiations take every tensor as dense [BH][T][D]
    TensorAt at_q, at_do, at_row_k, at_row_v, at_st_k, at_st_v;
    int H;
    const E *row_k, *row_v;    // [BH][T][D] "row" tensors: one row per wave and round (K2,V2 | K1,U)
    const E *st_k, *st_v;      // [BH][T][D] streamed tensors (K1,U | K2,V2) ...
    const E *st_kt, *st_vt;    // ... and their transposes [BH][D][Tp], zero padded
    const float *lse, *delta;  // [BH][T]
    E* dq;                     // written only by the WITH_DQ instantiation
    float *acc_k, *acc_v;      // [BH][T][D] fp32 gradients of row_k / row_v, zero on entry
    // general kernel only: the rows of a query tile are dealt out to `splits` workgroups; with more than
    // one, dQ / alpha is accumulated into acc_q (fp32, zero on entry) instead of being written to dq
    float* acc_q;
    int splits;
    // accumulate the row gradients (and a split dQ) as 64-bit fixed point with integer atomics (common.hpp: the
    // sums are bitwise the same whatever order the workgroups arrive in).  The accumulators then hold long long
    // where they otherwise hold float (twice the bytes, same element index); scale_parts / poison: see common.hpp
    int fixed_point;
    const unsigned* scale_parts;  // [BH][kScaleParts]
    unsigned* poison;             // [BH][T]
    unsigned bit_k, bit_v;        // poison bits of acc_k / acc_v
    int T, Tp, BH, nqt;
    int grid_tiles;  // query tiles the grid covers (nqt - 1 .. nqt - grid_tiles: tile 0 may be left to the fp32 kernel)
    float alpha;
    int causal;
    // windowed kernels only, in terms of the streamed index a and the row index b: (q, a, b) takes part
    // iff a, b <= q, q - a <= wa, q - b <= wb, b - a <= lab, a - b <= rab
    int wa, wb, lab, rab;
};

// the 16-bit kernels' accumulators resolve 2^-30 of the slice's max |dO| and cover sums up to 2^33 times it
constexpr int kFixedBias = 30;

// slice bh of a row-major tensor and its row pitch in elements (the compile-time D without SV)
template <bool SV, int D, typename E>
__device__ __forceinline__ const E* slice_of(const E* t, const TensorAt& at, int bh, int H, int T) {
    if constexpr (SV) return t + (size_t)(bh / H) * at.sb + (size_t)(bh % H) * at.sh;
    else return t + (size_t)bh * T * D;
}
template <bool SV, int D>
__device__ __forceinline__ unsigned pitch_of(const TensorAt& at) {
    if constexpr (SV) return at.st;
    else return (unsigned)D;
}

// scale of the fixed-point accumulators of slice bh (0: the accumulators are fp32)
template <typename E>
__device__ __forceinline__ float acc_scale(const BwdParams<E>& p, int bh) {
    return p.fixed_point ? fixed_scale_value(fixed_scale_field(p.scale_parts, bh, kFixedBias)) : 0.f;
}

}  // namespace tritt

#include "tdp_bwd_rows_general.hpp"
#include "tdp_bwd_rows_q16.hpp"
#include "tdp_f32_tiles.hpp"

namespace tritt {

// ------------------------------------------------------------------------------------------
// Written for launch 1 (rows = K2/V2 indexed by k, streamed = K1/U indexed by j); launch 2 is the
// same code with the two roles exchanged.
//
// Owner = 32 consecutive queries (the columns of every MFMA tile of the workgroup).  The eight
// waves take eight consecutive K2/V2 rows k per "round" (one k per wave), so a tile is
// (32 q) x (1 k), and sweep j in 64-row stages of K1 / U (and their transposes) shared by the
// workgroup.  Per round and wave, over the whole j sweep:
//   Yq[(q,k), :] = sum_j dS K1[j, :]        Tv[(q,k), :] = sum_j P U[j, :]
// and then
//   dQ[q]  += Yq (.) K2[k]                      (WITH_DQ: registers, all rounds; reduced over waves at the end)
//   dK2[k] += alpha * sum_q Yq (.) Q[q]         (sum over the tile's 32 rows in registers, then ONE
//   dV2[k] += sum_q Tv (.) dO[q]                 returnless fp32 atomic per element per (q-tile, k))
//
// The inner loop is laid out for latency: a wave that reads each MFMA operand from LDS just before
// the MFMA that uses it spends most of a step waiting for sixteen LDS round trips, and two waves
// per SIMD cannot hide that.  Here
//  * the eight row operands (K1 / U rows) of a step are read one step ahead, the eight transposed
//    operands (K1^T / U^T) right after the score products, under the exp2 / pack work;
//  * the gradient products of the first half of the registers are issued between the exp2 / pack
//    work of the second half;
//  * an invalid (q, j, k) gets -3e4 as C operand of the first score k-step, so its P is exactly 0
//    and interior and diagonal steps share one loop body: no branch around accumulator updates,
//    the accumulators stay in place;
//  * stages are fetched direct-to-LDS two ahead into three buffers and the workgroup barrier
//    sits in the middle of a stage: by then the next stage has landed for every wave, so its
//    first row operands are read during the second half and nothing waits at the stage boundary.
template <typename E, int D, bool WITH_DQ, bool SV>
__device__ __forceinline__ void tdp_bwd_rows_body(const BwdParams<E>& p, const int block) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = D / 32, BQ = 32, NW = 8, NTH = 64 * NW;
    constexpr int LDK = D + 8, LDF = D + 4;
    constexpr int TILE = 64 * 64;
    constexpr int NBUF = 3, LW = 4;  // stage buffers; direct loads per wave per stage
    static_assert(D == 64, "stages are four 64x64 tiles = 32 blocks of 1 KB, four per wave (D = 128 and windowed masks: tdp_bwd_rows_general_kernel)");

    extern __shared__ __align__(16) char smem[];
    E* sStage = reinterpret_cast<E*>(smem);  // [NBUF][4 tensors: K1, U, K1^T, U^T][TILE]
    E* sKr = sStage + NBUF * 4 * TILE;       // [2][8][D]  K2 rows of a round (one per wave), dense
    E* sVr = sKr + 2 * 8 * D;                // [2][8][D]  V2 rows
    // Q * alpha*log2(e) and dO as fp32 (operand build: one conversion and one multiply per product, and S is
    // rounded exactly as the forward rounded it)
    constexpr int LDQ = D + 4;
    float* sQb = reinterpret_cast<float*>(sVr + 2 * 8 * D);  // [BQ][LDQ]
    float* sOb = sQb + BQ * LDQ;                              // [BQ][LDQ]
    // dQ / alpha of the tile, summed over rounds: one slice per pair of waves, element (dt, i) of a
    // lane at [((dt * 4 + i / 4) * 64 + lane) * 4 + i % 4] (the accumulator layout, 16 bytes per access)
    float* sDQ = sOb + BQ * LDQ + (wave_of(threadIdx.x) >> 1) * (BQ * D);
    // Q and dO once more, in accumulator layout for the round epilogue: [dt][lane][i] = X[c_row(lane / 32, i)][32 dt + lane % 32]
    E* sQe = reinterpret_cast<E*>(sOb + BQ * LDQ + (NW / 2) * (BQ * D));
    E* sOe = sQe + DT * 64 * 16;

    const int xcd = block & 7;
    int slot = block >> 3;
    const int split = slot % p.splits;  // which share of the tile's rounds this workgroup walks (small grids)
    slot /= p.splits;
    int bh, order;
    if (!xcd_tile(p.BH, p.grid_tiles, slot, xcd, bh, order)) return;
    const int qt = p.nqt - 1 - order;  // heaviest query tiles first

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * p.Tp;
    const E* __restrict__ K1 = slice_of<SV, D>(p.st_k, p.at_st_k, bh, p.H, T);
    const E* __restrict__ U = slice_of<SV, D>(p.st_v, p.at_st_v, bh, p.H, T);
    const E* __restrict__ K2 = slice_of<SV, D>(p.row_k, p.at_row_k, bh, p.H, T);
    const E* __restrict__ V2 = slice_of<SV, D>(p.row_v, p.at_row_v, bh, p.H, T);
    const E* __restrict__ Qs = slice_of<SV, D>(p.q, p.at_q, bh, p.H, T);
    const E* __restrict__ Os = slice_of<SV, D>(p.d_o, p.at_do, bh, p.H, T);
    // row pitches in elements
    const unsigned pK1 = pitch_of<SV, D>(p.at_st_k), pU = pitch_of<SV, D>(p.at_st_v), pK2 = pitch_of<SV, D>(p.at_row_k),
                   pV2 = pitch_of<SV, D>(p.at_row_v), pQ = pitch_of<SV, D>(p.at_q), pO = pitch_of<SV, D>(p.at_do);
    const E* __restrict__ K1T = p.st_kt + tbase;
    const E* __restrict__ UT = p.st_vt + tbase;

    const int q0 = qt * BQ;
    const int qlast = min(T - 1, q0 + BQ - 1);
    const int jend = p.causal ? qlast : T - 1;  // last j (and last k) any query of the tile needs
    const int jfull = p.causal ? q0 : T - 1;    // keys / rows 0 .. jfull are valid for every column
    const int nst = jend / 64 + 1, nrounds = jend / 8 + 1;
    const bool dead_tail = (jend & 63) < 32;  // the last stage's second step lies past every query's last key
    const int per_split = (nrounds + p.splits - 1) / p.splits;
    const int m_lo = split * per_split, m_hi = min(nrounds, m_lo + per_split);
    if (m_lo >= m_hi) return;  // fewer rounds than shares (uniform over the workgroup, before any barrier)
    const int q = q0 + n;                        // this lane's column
    const bool q_ok = q < T;
    const int jq = p.causal ? min(q, T - 1) : T - 1;  // per-lane bound on j and k
    const float scale_log2 = p.alpha * kLog2e;
    const float fscale = acc_scale(p, bh);

    // stage loader: wave w fetches blocks 4*(w%2) .. +3 (8 rows each) of tensor w/2, direct to LDS
    const int tensor = wave >> 1;
    const bool rowmajor = tensor < 2;  // K1 / U: row = key j (read with permuted rows); else row = d
    const E* gsrc = uniform_ptr(tensor == 0 ? K1 : tensor == 1 ? U : tensor == 2 ? K1T : UT);
    // Per-lane byte offsets of the wave's four blocks inside a stage; the stage itself only moves
    // the (scalar) base.  Row-major tensors clamp rows past the end of the sequence (last stage of
    // a ragged T only): that path recomputes the offsets.
    const unsigned pitch = tensor == 0 ? pK1 : pU;  // of this wave's row-major tensor
    unsigned soff[LW];
    {
        const int pos = lane & 7, rr = lane >> 3;
#pragma unroll
        for (int c = 0; c < LW; ++c) {
            const int r = ((wave & 1) * 4 + c) * 8 + rr;
            soff[c] = rowmajor ? (unsigned)r * (pitch * 2) + ((pos ^ swz_perm(r)) * 16)
                               : (unsigned)r * p.Tp * 2 + ((pos ^ swz_seq(r)) * 16);
        }
    }
    auto issue_stage = [&](int st, int buf) {
        const int jb = st * 64;
        E* dst = sStage + (buf * 4 + tensor) * TILE + (wave & 1) * 4 * 512;
        if (rowmajor && jb + 63 > T - 1) {
            const int pos = lane & 7, rr = lane >> 3;
#pragma unroll
            for (int c = 0; c < LW; ++c) {
                const int r = ((wave & 1) * 4 + c) * 8 + rr;
                direct_load_16(gsrc, (unsigned)min(jb + r, T - 1) * (pitch * 2) + ((pos ^ swz_perm(r)) * 16), dst + c * 512);
            }
        } else {
            const E* sbase = gsrc + (size_t)jb * (rowmajor ? pitch : 1u);
#pragma unroll
            for (int c = 0; c < LW; ++c) direct_load_16(sbase, soff[c], dst + c * 512);
        }
    };
    auto issue_round = [&](int m, int buf) {  // waves 0, 1: K2 / V2 rows 8m .. 8m+7 (1 KB each)
        if (wave < 2) {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const unsigned off = (unsigned)min(m * 8 + (ln >> 3), T - 1) * ((wave ? pV2 : pK2) * 2) + (ln & 7) * 16;
            direct_load_16(uniform_ptr(wave ? V2 : K2), off, (wave ? sVr : sKr) + buf * 8 * D);
        }
    };

    // prologue: Q / dO tiles in both forms, first round, first three stages (the j sweep repeats
    // every round, so stage numbers simply cycle: stage of running index x is x mod nst)
    for (int idx = tid; idx < BQ * D; idx += NTH) {
        const int r = idx / D, d = idx % D;
        const unsigned row = (unsigned)min(q0 + r, T - 1);
        const E qv = Qs[(size_t)row * pQ + d], ov = Os[(size_t)row * pO + d];
        sQb[r * LDQ + d] = (float)qv * scale_log2;
        sOb[r * LDQ + d] = (float)ov;
    }
    for (int idx = tid; idx < DT * 64 * 16; idx += NTH) {
        const int i = idx & 15, ln = (idx >> 4) & 63, dt = idx >> 10;
        const unsigned row = (unsigned)min(q0 + c_row(ln >> 5, i), T - 1);
        sQe[idx] = Qs[(size_t)row * pQ + dt * 32 + (ln & 31)];
        sOe[idx] = Os[(size_t)row * pO + dt * 32 + (ln & 31)];
    }
    if constexpr (WITH_DQ) {
        float* all = sOb + BQ * LDQ;
        for (int idx = tid; idx < (NW / 2) * BQ * D; idx += NTH) all[idx] = 0.f;
    }
    issue_round(m_lo, m_lo & 1);
    issue_stage(0, 0);
    issue_stage(1 % nst, 1);
    barrier_keep_loads<0>();  // stages 0 and 1 and the first round have landed for every wave

    // per-column constants that enter the score products as C operands; a column past the end of
    // the sequence gets a huge LSE so that its P underflows to exactly 0
    const float lse2 = q_ok ? p.lse[(size_t)bh * T + q] * kLog2e : 3.0e4f;  // representable in fp16 too
    const float delta = q_ok ? p.delta[(size_t)bh * T + q] : 0.f;
    // C operands of the first k-step of S and dP: -LSE2[q] / -Delta[q] in every register of the lane
    // (the columns of a tile are the queries).  Opaque, so that they stay in registers.
    f32x16 init_s, init_dp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        init_s[i] = -lse2;
        init_dp[i] = -delta;
    }
    asm volatile("" : "+v"(init_s), "+v"(init_dp));
    const int krow_off = key_of_row(n);
    const int fperm = swz_perm(krow_off), fseq = swz_seq(n);

    // dQ[q] += Yq (.) K2[k] once per round.  A register tile per wave would cost 32 registers in a
    // loop that has none to spare, so the running sum lives in LDS: the two waves of a pair add
    // their round's tile to the pair's slice one after the other, the even wave before the
    // round-end barrier, the odd wave after it.
    // row operands (K1 / U rows in MFMA A layout) of the step about to run
    v8 ak[KS], au[KS];
    auto load_rows = [&](int buf, int half) {
        const E* sK1 = sStage + (buf * 4 + 0) * TILE;
        const E* sU = sStage + (buf * 4 + 1) * TILE;
        const int rowoff = (half * 32 + krow_off) * 64;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            ak[ks] = *reinterpret_cast<const v8*>(sK1 + rowoff + (((ks * 2 + g) ^ fperm) * 8));
            au[ks] = *reinterpret_cast<const v8*>(sU + rowoff + (((ks * 2 + g) ^ fperm) * 8));
        }
    };
    load_rows(0, 0);

    const bool late = (wave >> 2) & 1;  // second wave of its SIMD (waves w and w + 4 share one)
    int gstage = 0;          // running stage index; buffer = gstage % NBUF
    int st_ahead = 2 % nst;  // stage number of running index gstage + 2
    for (int m = m_lo; m < m_hi; ++m) {
        const int mb = m & 1;
        const int k = m * 8 + wave;  // this wave's K2/V2 row

        v8 bq[KS], bg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int off = ks * 16 + g * 8;
            const v8 kv = *reinterpret_cast<const v8*>(sKr + (mb * 8 + wave) * D + off);
            const v8 vv = *reinterpret_cast<const v8*>(sVr + (mb * 8 + wave) * D + off);
            const float4 qa = *reinterpret_cast<const float4*>(sQb + n * LDQ + off);
            const float4 qb = *reinterpret_cast<const float4*>(sQb + n * LDQ + off + 4);
            const float4 da = *reinterpret_cast<const float4*>(sOb + n * LDQ + off);
            const float4 db = *reinterpret_cast<const float4*>(sOb + n * LDQ + off + 4);
            const float qv[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            const float dv[8] = {da.x, da.y, da.z, da.w, db.x, db.y, db.z, db.w};
            v8 a, b;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const v2 pa = M::pack((float)kv[e] * qv[e], (float)kv[e + 1] * qv[e + 1]);
                const v2 pb = M::pack((float)vv[e] * dv[e], (float)vv[e + 1] * dv[e + 1]);
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
            const E* sK1T = sStage + (sb * 4 + 2) * TILE;
            const E* sUT = sStage + (sb * 4 + 3) * TILE;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int jb = st * 64 + half * 32;
                // wave-uniform: some (q, j, k) of this step is invalid
                const bool need_mask = (k > jfull) || (jb + 31 > jfull);
                f32x16 s, dp;
                __builtin_amdgcn_sched_barrier(0);
                // Wave priority: low while this wave issues the score products (eight MFMAs and nothing else), high for
                // the rest of the step.  The other wave of the SIMD is half a step away, in its exp2 / pack work: served
                // first, its vector instructions go out at once and these MFMAs fill the slots between them, instead of the
                // older wave's MFMAs holding the issue port while the vector work waits (backward 11.28 -> 11.07 ms).
                __builtin_amdgcn_s_setprio(0);
                // S starts from -LSE2[q] and dP from -Delta[q] (C operand of the first k-step); where
                // (q, j, k) is invalid S starts from -3e4 instead.  Element i of a lane is key
                // jb + key_of(0, i) + 8 g.
                if (need_mask) {
                    const int lim = (k <= jq) ? jq - jb - 8 * g : -1;
                    f32x16 c;
#pragma unroll
                    for (int i = 0; i < 16; ++i) c[i] = key_of(0, i) <= lim ? -lse2 : -3.0e4f;
                    s = M::mma(ak[0], bq[0], c);
                } else {
                    s = M::mma(ak[0], bq[0], init_s);
                }
                dp = M::mma(au[0], bg[0], init_dp);
                __builtin_amdgcn_sched_barrier(0);
                if (half == 1) {
                    // the buffer two stages ahead was last read in the previous stage, and every wave is
                    // past that (this stage's barrier was crossed in the first half): fetch it now
                    if (st == 0 && m + 1 < m_hi) issue_round(m + 1, mb ^ 1);  // older than the stage loads
                    issue_stage(st_ahead, (gstage + 2) % NBUF);
                    st_ahead = st_ahead + 1 < nst ? st_ahead + 1 : 0;
                }
                __builtin_amdgcn_sched_barrier(0);
                // a step past every query's last key (the second half of the last stage, for every other tile) has
                // S = -3e4 from the C operand above, so P = dS = 0 whatever the other k-steps would add: they are skipped
                const bool dead = half == 1 && dead_tail && st == nst - 1;
                if (!dead) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        if (ks > 0) s = M::mma(ak[ks], bq[ks], s);
                        if (ks > 0) dp = M::mma(au[ks], bg[ks], dp);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                // (the second wave of the SIMD one level above the first, so that the two never tie: another 0.8 %)
                if (late) __builtin_amdgcn_s_setprio(2);
                else __builtin_amdgcn_s_setprio(1);
                // transposed operands of the gradient products: they land under the exp2 / pack work
                v8 bt[DT][2], bk[DT][2];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int toff = (dt * 32 + n) * 64 + (((half * 4 + h * 2 + g) ^ fseq) * 8);
                        bt[dt][h] = *reinterpret_cast<const v8*>(sUT + toff);
                        bk[dt][h] = *reinterpret_cast<const v8*>(sK1T + toff);
                    }
                __builtin_amdgcn_sched_barrier(0);
                if (half == 0 && late) barrier_keep_loads<0>();  // see below
                __builtin_amdgcn_sched_barrier(0);
                v8 pa[2], da[2];
                // register pair r (0..7):  P = exp2(S), dS = P dP, both packed to 16 bit
                auto softmax_pair = [&](int r) {
                    const int h = r >> 2, e = 2 * (r & 3), i = h * 8 + e;
                    const float p0 = fast_exp2(s[i]), p1 = fast_exp2(s[i + 1]);
                    const v2 pp = M::pack(p0, p1);
                    const v2 dd = M::pack(p0 * dp[i], p1 * dp[i + 1]);
                    pa[h][e] = pp[0]; pa[h][e + 1] = pp[1];
                    da[h][e] = dd[0]; da[h][e + 1] = dd[1];
                };
                static_assert(DT == 2, "interleave written for D = 64");
                if (!dead) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) softmax_pair(r);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if ((r & 1) == 0) accT[r >> 1] = M::mma(pa[0], bt[r >> 1][0], accT[r >> 1]);
                        else accQ[r >> 1] = M::mma(da[0], bk[r >> 1][0], accQ[r >> 1]);
                        __builtin_amdgcn_sched_barrier(0);
                        softmax_pair(4 + r);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                // the row operands are dead: read those of the next step (second half of this stage,
                // or first half of the next one, which has landed for everyone since the barrier)
                load_rows(half == 0 ? sb : (gstage + 1) % NBUF, half ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                if (!dead) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if ((r & 1) == 0) accT[r >> 1] = M::mma(pa[1], bt[r >> 1][1], accT[r >> 1]);
                        else accQ[r >> 1] = M::mma(da[1], bk[r >> 1][1], accQ[r >> 1]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                // The stage's one workgroup barrier: the next stage has landed for every wave, everyone is
                // done with the previous one.  The two waves of a SIMD cross it at different points of
                // their step (the first after its first step, the second in the middle of it, above):
                // waves that leave a barrier in the same phase run score products together and exp2
                // work together, with the other pipe idle; half a step apart, one wave's matrix phase
                // runs under the other's vector phase.
                if (half == 0 && !late) barrier_keep_loads<0>();
            }
        }

        // ---- round epilogue (rows of the accumulators = the 32 queries, column = d) ---------------
        // columns 32 dt .. + 31 of the slice += Yq (.) K2[k]; dt at compile time (a run-time choice of registers would be
        // indexed through M0, which the direct loads own)
        [[maybe_unused]] auto add_dq = [&](auto dt_c) {
            constexpr int dt = decltype(dt_c)::value;
            {
                const float kd = (float)sKr[(mb * 8 + wave) * D + dt * 32 + n];
#pragma unroll
                for (int i4 = 0; i4 < 4; ++i4) {
                    float4* slot = reinterpret_cast<float4*>(sDQ + ((dt * 4 + i4) * 64 + lane) * 4);
                    float4 v = *slot;
                    v.x += accQ[dt][i4 * 4] * kd; v.y += accQ[dt][i4 * 4 + 1] * kd;
                    v.z += accQ[dt][i4 * 4 + 2] * kd; v.w += accQ[dt][i4 * 4 + 3] * kd;
                    *slot = v;
                }
            }
        };
        if (k <= jend) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = dt * 32 + n;
                [[maybe_unused]] const float kd = (float)sKr[(mb * 8 + wave) * D + d];
                float sk = 0.f, sv = 0.f;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const v8 qv = *reinterpret_cast<const v8*>(sQe + (dt * 64 + lane) * 16 + h * 8);
                    const v8 ov = *reinterpret_cast<const v8*>(sOe + (dt * 64 + lane) * 16 + h * 8);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        sk += accQ[dt][h * 8 + e] * (float)qv[e];
                        sv += accT[dt][h * 8 + e] * (float)ov[e];
                    }
                }
                sk += __shfl_xor(sk, 32, 64);
                sv += __shfl_xor(sv, 32, 64);
                if (g == 0) {
                    unsigned* prow = p.poison + (size_t)bh * T + k;
                    shared_add(p.acc_k, base + (size_t)k * D + d, sk * p.alpha, fscale, prow, p.bit_k);
                    shared_add(p.acc_v, base + (size_t)k * D + d, sv, fscale, prow, p.bit_v);
                }
            }
        }
        // The two waves of a pair add their tiles to the pair's slice half and half: before the barrier the even wave
        // its columns 0-31 and the odd wave its columns 32-63, after it the other halves.  (One wave before and one
        // after puts two chains of eight dependent LDS round trips on the workgroup's path per round instead of two of four.)
        if constexpr (WITH_DQ) {
            if (k <= jend) {
                if (wave & 1) add_dq(std::integral_constant<int, 1>{});
                else add_dq(std::integral_constant<int, 0>{});
            }
        }
        // all waves are done with this round's K2/V2 rows; the next round's have landed: they are older than the newest
        // stage's loads, the only ones allowed to stay in flight (a tile of a single stage issues both in its one step)
        barrier_keep_loads<LW>();
        if constexpr (WITH_DQ) {
            if (k <= jend) {
                if (wave & 1) add_dq(std::integral_constant<int, 0>{});
                else add_dq(std::integral_constant<int, 1>{});
            }
        }
    }
    wait_vmcnt<0>();  // the stages fetched ahead land in the buffers reused below
    __syncthreads();

    if constexpr (WITH_DQ) {
        // ---- dQ: sum the pairs' slices; thread (wave, lane) owns accumulator registers 4*(wave%4) .. +3
        // of d-tile wave/4, i.e. four consecutive query rows of column d
        const float* all = sOb + BQ * LDQ;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int sl = 0; sl < NW / 2; ++sl) {
            const float4 x = *reinterpret_cast<const float4*>(all + sl * (BQ * D) + (wave * 64 + lane) * 4);
            v.x += x.x; v.y += x.y; v.z += x.z; v.w += x.w;
        }
        const int d = (wave >> 2) * 32 + n, r0 = c_row(g, (wave & 3) * 4);
        const float out[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (q0 + r0 + e < T) {
                const size_t off = base + (size_t)(q0 + r0 + e) * D + d;
                if (p.splits > 1)  // scaled by alpha when converted
                    shared_add(p.acc_q, off, out[e], fscale, p.poison + (size_t)bh * T + q0 + r0 + e, kPoisonDQ);
                else p.dq[off] = (E)(out[e] * p.alpha);
            }
    }
}

template <typename E, int D, bool WITH_DQ, bool SV = false>
__global__ __launch_bounds__(512) void tdp_bwd_rows_kernel(BwdParams<E> p) {
    tdp_bwd_rows_body<E, D, WITH_DQ, SV>(p, blockIdx.x);
}

// The same grid together with the fp32 workgroups of query tile 0 (tdp_f32_tiles.hpp: both roles, one workgroup per
// round of eight rows; t0_x * 2 * rounds of them).  As a launch of their own they are 64 short workgroups between two
// launches that fill the chip, 30 us in which most of it idles.  Here they come after the main blocks, beside the
// last and lightest tiles of the launch (t0_first = 0: large grids, whose heavy tiles should start at once), or
// before them (small grids: the main blocks are as short as these, and a latency-bound workgroup that starts last
// is the launch's tail).  They add to the same accumulators as every other workgroup, in fixed point, so the order
// changes nothing.
template <typename E, int D, bool WITH_DQ, bool SV>
__global__ __launch_bounds__(512) void tdp_bwd_rows_tile0_kernel(BwdParams<E> p, F32BwdParams<E> r0, F32BwdParams<E> r1,
                                                                 int roles_mask, int main_blocks, int t0_x, int t0_first) {
    const int t0_blocks = t0_x * 2 * r0.split_rounds;
    const int block = (int)blockIdx.x - (t0_first ? t0_blocks : 0);  // main blocks: 0 .. main_blocks - 1
    if (block >= 0 && block < main_blocks) {
        tdp_bwd_rows_body<E, D, WITH_DQ, SV>(p, block);
    } else {
        const int extra = t0_first ? (int)blockIdx.x : block - main_blocks;
        f32_tile0_block<E, D, D>(r0, r1, roles_mask, extra / t0_x, extra % t0_x);
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
                                                       float* __restrict__ zero_b, float* __restrict__ zero_c,
                                                       float* __restrict__ zero_d, float* __restrict__ zero_e, int T,
                                                       int Tp, int D, int zero_width,
                                                       unsigned* __restrict__ scale_parts,
                                                       unsigned* __restrict__ poison,
                                                       const E* __restrict__ o_res, int H, TensorAt at_v1,
                                                       TensorAt at_k1, TensorAt at_k2, TensorAt at_v2, TensorAt at_do) {
    // v1, k1, k2, v2 and d_o lie where the caller has them (H heads per batch entry, strides in elements; a dense
    // call passes H = 1 and dense strides); everything else is dense
    const int bh = blockIdx.y, j0 = blockIdx.x * 64;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * Tp;
    const int b_ = bh / H, h_ = bh % H;
    auto slice = [&](const E* t, const TensorAt& at) { return t + (size_t)b_ * at.sb + (size_t)h_ * at.sh; };
    v1 = slice(v1, at_v1); k1 = slice(k1, at_k1); k2 = slice(k2, at_k2); v2 = slice(v2, at_v2); d_o = slice(d_o, at_do);
    if (scale_parts) {
        // fixed-point accumulators: clear the poison words of this block's rows; the first blocks of a slice
        // also leave the partial maxima of |dO| that fix the slice's scale (part s = 64-row blocks s, s + 8, ...)
        __shared__ unsigned red[4];
        if (threadIdx.x < 64 && j0 + threadIdx.x < T) poison[(size_t)bh * T + j0 + threadIdx.x] = 0;
        for (int part = blockIdx.x; part < kScaleParts; part += gridDim.x) {
            unsigned m = 0;
            for (int r0 = part * 64; r0 < T; r0 += kScaleParts * 64)
                m = max(m, block_absmax_bits<E>(d_o + (size_t)r0 * at_do.st, (size_t)min(64, T - r0) * D / 8, red, D / 8, at_do.st));
            if (threadIdx.x == 0) scale_parts[bh * kScaleParts + part] = m;
        }
    }
    // two tiles at a time (static LDS stays under 64 KB at D = 128): their loads are in flight together
    constexpr int kTile = 64 * (128 + 2);
    __shared__ E tiles[2 * kTile];
    transpose_load<E, true>(v1, u + base, tiles, j0, T, D, at_v1.st);
    transpose_load<E, false>(k1, nullptr, tiles + kTile, j0, T, D, at_k1.st);
    __syncthreads();
    transpose_store<E>(ut + tbase, tiles, j0, Tp, D);
    transpose_store<E>(k1t + tbase, tiles + kTile, j0, Tp, D);
    __syncthreads();
    transpose_load<E, false>(k2, nullptr, tiles, j0, T, D, at_k2.st);
    transpose_load<E, false>(v2, nullptr, tiles + kTile, j0, T, D, at_v2.st);
    __syncthreads();
    transpose_store<E>(k2t + tbase, tiles, j0, Tp, D);
    transpose_store<E>(v2t + tbase, tiles + kTile, j0, Tp, D);
    // the accumulators: zero_width 4-byte words per row (D floats, or D 64-bit fixed-point sums)
    const float4 z4 = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int idx = threadIdx.x; idx < 64 * (zero_width / 4); idx += 256) {
        const int j = j0 + idx / (zero_width / 4);
        if (j < T) {
            const size_t off = ((size_t)bh * T + j) * zero_width + (idx % (zero_width / 4)) * 4;
            *reinterpret_cast<float4*>(zero_a + off) = z4;
            *reinterpret_cast<float4*>(zero_b + off) = z4;
            *reinterpret_cast<float4*>(zero_c + off) = z4;
            *reinterpret_cast<float4*>(zero_d + off) = z4;
            if (zero_e) *reinterpret_cast<float4*>(zero_e + off) = z4;
        }
    }
    // Delta[j] = dO[j] . O[j]: the D / 8 lanes that hold a row's 16-byte pieces sit next to each other
    typedef __attribute__((ext_vector_type(8))) E e8;
    const int cpr = D / 8;
    for (int idx = threadIdx.x; idx < 64 * cpr; idx += 256) {
        const int j = j0 + idx / cpr, c = idx % cpr;
        float part = 0.f;
        if (j < T) {
            const size_t off = base + (size_t)j * D + c * 8;
            const e8 a = *reinterpret_cast<const e8*>(o + off);
            const e8 b = *reinterpret_cast<const e8*>(d_o + (size_t)j * at_do.st + c * 8);
            if (o_res) {  // split operands: the output to 16 mantissa bits (rounded value + rounding residual)
                const e8 r = *reinterpret_cast<const e8*>(o_res + off);
#pragma unroll
                for (int e = 0; e < 8; ++e) part += ((float)a[e] + (float)r[e]) * (float)b[e];
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) part += (float)a[e] * (float)b[e];
            }
        }
        for (int off = cpr >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
        if (c == 0 && j < T) delta[(size_t)bh * T + j] = part;
    }
}

// fp32 accumulators -> output tensors; dV1 = dU * SiLU'(V1)
template <typename E>
__global__ __launch_bounds__(256) void bwd_finish_kernel(const float* __restrict__ dk1acc,
                                                         const float* __restrict__ duacc,
                                                         const float* __restrict__ dk2acc,
                                                         const float* __restrict__ dv2acc,
                                                         const float* __restrict__ dqacc, float alpha,
                                                         E* __restrict__ dq, const E* __restrict__ v1,
                                                         E* __restrict__ dk1, E* __restrict__ dv1, E* __restrict__ dk2,
                                                         E* __restrict__ dv2, size_t n, int fixed_point,
                                                         const float* __restrict__ dq0acc, int T, int D,
                                                         const unsigned* __restrict__ scale_parts,
                                                         const unsigned* __restrict__ poison, int H, TensorAt at_v1) {
    // a null output is a gradient the caller does not want; v1 lies where the caller has it (see bwd_prep_kernel)
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t row = i / D, t = row % T;
        double inv = 0.0;
        unsigned bad = 0;
        if (fixed_point) {
            inv = fixed_scale_inverse(fixed_scale_field<false>(scale_parts, (int)(row / T), kFixedBias));
            bad = poison[row];
        }
        auto value = [&](const float* acc, size_t at, unsigned bit) {
            if (!fixed_point) return acc[at];
            if (bad & bit) return __builtin_nanf("");
            return (float)((double)reinterpret_cast<const long long*>(acc)[at] * inv);
        };
        if (dk1) dk1[i] = (E)value(dk1acc, i, kPoisonDK1);
        if (dv1) {
            const size_t bh = row / T;
            const E x = v1[(bh / H) * at_v1.sb + (bh % H) * at_v1.sh + t * at_v1.st + i % D];
            dv1[i] = (E)(value(duacc, i, kPoisonDU) * silu_grad_f((float)x));
        }
        if (dk2) dk2[i] = (E)value(dk2acc, i, kPoisonDK2);
        if (dv2) dv2[i] = (E)value(dv2acc, i, kPoisonDV2);
        if (dqacc && dq) dq[i] = (E)(value(dqacc, i, kPoisonDQ) * alpha);
        // query tile 0 was summed over its rounds in a [BH][32][D] accumulator
        if (dq0acc && dq && t < 32) dq[i] = (E)(value(dq0acc, (row / T * 32 + t) * D + i % D, kPoisonDQ) * alpha);
    }
}

struct BwdLayout {
    size_t u, ut, k1t, k2t, v2t, delta, lse_f32, delta_f32, dq0acc, scale_parts, poison, dk1acc, duacc, dk2acc, dv2acc,
        dqacc, total;
};
static BwdLayout bwd_layout(int BH, int T, int D, bool fixed_point) {
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
    l.lse_f32 = take((size_t)BH * T * 4);    // fp32 tiles of the backward: their rows' LSE and Delta in fp32
    l.delta_f32 = take(std::max((size_t)BH * T, (size_t)BH * 32 * 4 * 3) * 4);
    l.dq0acc = take((size_t)BH * 32 * D * 8);  // dQ / alpha of query tile 0, summed over its rounds
    l.scale_parts = take((size_t)BH * kScaleParts * 4);  // fixed point: see common.hpp
    l.poison = take((size_t)BH * T * 4);
    const size_t acc = fixed_point ? 8 : 4;
    l.dk1acc = take(n * acc);
    l.duacc = take(n * acc);
    l.dk2acc = take(n * acc);
    l.dv2acc = take(n * acc);
    l.dqacc = take(n * acc);  // used when the rows of a query tile are split over workgroups (small grids)
    l.total = (off + 255) & ~size_t(255);
    return l;
}

// SV: the caller's tensors are strided views, read where they lie (the kernels' SV instantiations)
template <typename E, int D, bool SV>
static hipError_t launch_bwd(const MfmaBwdArgs& a, hipStream_t st) {
    const int Tp = (a.T + 63) / 64 * 64;
    const BwdLayout l = bwd_layout(a.BH, a.T, D, a.deterministic);
    char* ws = static_cast<char*>(a.workspace);
    const E *u = (const E*)(ws + l.u), *ut = (const E*)(ws + l.ut), *k1t = (const E*)(ws + l.k1t);
    const E *k2t = (const E*)(ws + l.k2t), *v2t = (const E*)(ws + l.v2t);
    float *dk1acc = (float*)(ws + l.dk1acc), *duacc = (float*)(ws + l.duacc);
    float *dk2acc = (float*)(ws + l.dk2acc), *dv2acc = (float*)(ws + l.dv2acc);

    // A workgroup owns a 32-query tile and walks all of its rows.  When that leaves most of the chip idle, or
    // ends in a long tail (few heads, short sequences), the rows of a tile are dealt out to several
    // workgroups, and dQ is accumulated in fp32 like the row gradients.
    const int tiles = 8 * ((a.BH + 7) / 8) * ((a.T + 31) / 32);
    int splits = 1;
    if (tiles < 1024) splits = std::min(16, (1024 + tiles - 1) / tiles);
    // a few waves of long tiles: the last tiles of each head are the costliest (the work of a tile grows with the
    // square of its position), and halving them shortens the tail by about 1 % (measured: B=4 H=8 T=1024, 2048)
    else if (tiles < 4096 && a.T >= 1024) splits = 2;
    if (knobs().bwd_splits > 0) splits = std::min(16, knobs().bwd_splits);  // tuning sweeps
    float* dqacc = splits > 1 ? (float*)(ws + l.dqacc) : nullptr;

    hipLaunchKernelGGL(bwd_prep_kernel<E>, dim3(Tp / 64, a.BH), dim3(256), 0, st, (const E*)a.v1, (const E*)a.k1,
                       (const E*)a.k2, (const E*)a.v2, (const E*)a.o, (const E*)a.d_o, (E*)(ws + l.u),
                       (E*)(ws + l.ut), (E*)(ws + l.k1t), (E*)(ws + l.k2t), (E*)(ws + l.v2t),
                       (float*)(ws + l.delta), dk1acc, duacc, dk2acc, dv2acc, dqacc, a.T, Tp, D,
                       a.deterministic ? 2 * D : D, a.deterministic ? (unsigned*)(ws + l.scale_parts) : nullptr,
                       (unsigned*)(ws + l.poison),
                       a.split ? (const E*)a.o + (size_t)a.BH * a.T * D : (const E*)nullptr, SV ? a.H : 1,
                       SV ? a.at_v1 : dense_at(1, a.T, D), SV ? a.at_k1 : dense_at(1, a.T, D),
                       SV ? a.at_k2 : dense_at(1, a.T, D), SV ? a.at_v2 : dense_at(1, a.T, D),
                       SV ? a.at_do : dense_at(1, a.T, D));

    BwdParams<E> p;
    p.H = SV ? a.H : 1;
    const TensorAt at_u = dense_at(p.H, a.T, D);  // SiLU(V1), in the workspace
    p.at_q = a.at_q; p.at_do = a.at_do;
    p.q = (const E*)a.q; p.d_o = (const E*)a.d_o;
    p.lse = a.lse; p.delta = (const float*)(ws + l.delta);
    p.dq = (E*)a.dq;
    p.T = a.T; p.Tp = Tp; p.BH = a.BH; p.nqt = (a.T + 31) / 32;
    p.alpha = a.alpha; p.causal = a.causal;
    p.acc_q = dqacc; p.splits = splits; p.fixed_point = a.deterministic ? 1 : 0;
    p.scale_parts = (const unsigned*)(ws + l.scale_parts); p.poison = (unsigned*)(ws + l.poison);

    // D = 64, full windows: three stage buffers of four 64x64 tiles, two rounds of 8 K2 / V2 rows, the Q and dO
    // tiles (twice: operand and epilogue layout), four dQ slices.  Otherwise: tdp_bwd_rows_general.hpp
    size_t smem;
    void (*kern_dq)(BwdParams<E>);
    void (*kern_nodq)(BwdParams<E>);
    int nthreads = 512, col_parts = 1;
    bool plain64 = false;  // the D = 64 kernel of this file
    if constexpr (D == 32) {
        // one shape, the banded instantiation for every mask (full windows are windows of T)
        smem = bwdg_smem(32, 8, 32, true);
        kern_dq = tdp_bwd_rows_general_kernel<E, 32, true, 8, 32, true, false, SV>;
        kern_nodq = tdp_bwd_rows_general_kernel<E, 32, false, 8, 32, true, false, SV>;
        if (a.split) {
            kern_dq = tdp_bwd_rows_general_kernel<E, 32, true, 8, 32, true, true, SV>;
            kern_nodq = tdp_bwd_rows_general_kernel<E, 32, false, 8, 32, true, true, SV>;
        }
    } else if (a.split) {
        // split operands: the general kernel (banded instantiation: full windows are windows of T)
        if constexpr (D == 64) {
            smem = bwdg_smem(64, 8, 64, true);
            kern_dq = tdp_bwd_rows_general_kernel<E, 64, true, 8, 64, true, true, SV>;
            kern_nodq = tdp_bwd_rows_general_kernel<E, 64, false, 8, 64, true, true, SV>;
            if (!a.windowed) {
                kern_dq = tdp_bwd_rows_general_kernel<E, 64, true, 8, 64, false, true, SV>;
                kern_nodq = tdp_bwd_rows_general_kernel<E, 64, false, 8, 64, false, true, SV>;
            }
        } else {
            return hipErrorInvalidValue;
        }
    } else if (a.windowed && D == 128 && knobs().bwd128_variant != 8) {
        // the 16-query kernel (tdp_bwd_rows_q16.hpp), banded instantiation
        if constexpr (D == 128) {
            smem = bwd_q16_smem();
            kern_dq = tdp_bwd_rows_q16_kernel<E, true, true, SV>;
            kern_nodq = tdp_bwd_rows_q16_kernel<E, false, true, SV>;
        }
    } else if (a.windowed) {
        smem = bwdg_smem(D, 8, 64, true);
        kern_dq = tdp_bwd_rows_general_kernel<E, (D < 64 ? 64 : D), true, 8, 64, true, false, SV>;
        kern_nodq = tdp_bwd_rows_general_kernel<E, (D < 64 ? 64 : D), false, 8, 64, true, false, SV>;
        col_parts = D / 64;
    } else if constexpr (D == 128) {
        // Default: 16 queries per wave on 16x16x32 tiles, every gradient column in one wave, S and dP formed once
        // (tdp_bwd_rows_q16.hpp).  The two 32-query shapes stay selectable (TRITT_TUNE_BWD128_WAVES = 8 | 4,
        // TRITT_BWD128_VARIANT=w8 | w4): two waves per SIMD with 64 gradient columns per workgroup (S and dP
        // computed by both column halves), or one wave per SIMD with all 128 columns.
        const int variant = knobs().bwd128_variant;
        if (variant != 4 && variant != 8) {
            smem = bwd_q16_smem();
            kern_dq = tdp_bwd_rows_q16_kernel<E, true, false, SV>;
            kern_nodq = tdp_bwd_rows_q16_kernel<E, false, false, SV>;
        } else if (variant == 8) {
            smem = bwdg_smem(128, 8, 64, true);
            kern_dq = tdp_bwd_rows_general_kernel<E, 128, true, 8, 64, false, false, SV>;
            kern_nodq = tdp_bwd_rows_general_kernel<E, 128, false, 8, 64, false, false, SV>;
            col_parts = 2;
        } else {
            smem = bwdg_smem(128, 4, 128, true);
            kern_dq = tdp_bwd_rows_general_kernel<E, 128, true, 4, 128, false, false, SV>;
            kern_nodq = tdp_bwd_rows_general_kernel<E, 128, false, 4, 128, false, false, SV>;
            nthreads = 256;
        }
    } else {
        smem = 2 * (size_t)(3 * 4 * 64 * 64 + 2 * 2 * 8 * 64 + 2 * (64 / 32) * 64 * 16) +
               4 * (size_t)(2 * 32 * (64 + 4) + 4 * 32 * 64);
        kern_dq = tdp_bwd_rows_kernel<E, 64, true, SV>;
        kern_nodq = tdp_bwd_rows_kernel<E, 64, false, SV>;
        plain64 = true;
    }
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern_dq), smem); e != hipSuccess) return e;
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern_nodq), smem); e != hipSuccess) return e;
    const bool want_q = a.dq != nullptr, want_k2 = a.dk2 || a.dv2, want_k1 = a.dk1 || a.dv1;
    // Under a causal mask the first query tile goes through the fp32 kernel (tdp_f32_mfma.hip): its softmax rows
    // are nearly one-hot, and dS = P (dP - Delta) then cancels two numbers whose 16-bit operand rounding the
    // kernels here cannot resolve (query 0 has a gradient of exactly zero in dQ).  The kernels below start at
    // tile 1: the grid simply has one tile less, and the heaviest-first numbering never reaches tile 0.
    // A windowed mask that leaves a query no more than about a thousand (j, k) pairs makes every row like that:
    // then all query tiles take the fp32 kernel (the work of such masks is small: T times the pair count).
    const bool first_in_f32 = a.causal != 0;
    const long long pairs = (long long)(a.k2_window + 1) * std::min(a.k1_window + 1, a.kk_left + a.kk_right + 1);
    const bool all_in_f32 = first_in_f32 && a.windowed && pairs <= 1024 && !a.split;
    // tile 0's backward workgroups ride at the end of the first rows launch below where that is the D = 64 kernel
    // (tdp_bwd_rows_tile0_kernel); otherwise they are a launch of their own
    bool fuse_tile0 = false;
    [[maybe_unused]] F32BwdParams<E> t0_r0{}, t0_r1{};
    [[maybe_unused]] int t0_roles = 0, t0_rounds = 0;
    if (first_in_f32) {
        FirstTileArgs f{};
        f.q = a.q; f.d_o = a.d_o; f.k1 = a.k1; f.u = u; f.k2 = a.k2; f.v2 = a.v2;
        f.H = SV ? a.H : 0; f.at_q = a.at_q; f.at_do = a.at_do; f.at_k1 = a.at_k1; f.at_k2 = a.at_k2; f.at_v2 = a.at_v2;
        f.lse_f32 = (float*)(ws + l.lse_f32); f.delta_f32 = (float*)(ws + l.delta_f32);
        f.dq0_acc = ws + l.dq0acc;
        f.dq = a.dq; f.acc_k2 = dk2acc; f.acc_v2 = dv2acc; f.acc_k1 = dk1acc; f.acc_u = duacc; f.acc_q = dqacc;
        f.scale_parts = a.deterministic ? p.scale_parts : nullptr; f.poison = p.poison; f.scale_bias = kFixedBias;
        f.BH = a.BH; f.T = a.T; f.D = D; f.is_bf16 = a.is_bf16;
        f.alpha = a.alpha; f.causal = a.causal;
        f.k1_window = a.k1_window; f.k2_window = a.k2_window; f.kk_left = a.kk_left; f.kk_right = a.kk_right;
        f.want_q = want_q; f.want_k2 = want_k2; f.want_k1 = want_k1;
        f.tiles = all_in_f32 ? p.nqt : 1;
        f.round_parts = (dqacc || !want_q) ? std::min(splits, f32_round_parts(a.BH, a.T)) : 1;
        if constexpr (D == 64) {
            if (plain64 && !all_in_f32 && p.nqt > 1 && (want_q || want_k2 || want_k1)) {
                if (hipError_t e = tile0_prepare<E, 64>(f, st, t0_r0, t0_r1, t0_roles, t0_rounds); e != hipSuccess) return e;
                fuse_tile0 = true;
            }
        }
        if (!fuse_tile0)
            if (hipError_t e = f32_mfma_tdp_bwd_first_tile(f, st); e != hipSuccess) return e;
    }
    const int tiles_here = all_in_f32 ? 0 : p.nqt - (first_in_f32 ? 1 : 0);
    p.grid_tiles = std::max(tiles_here, 1);  // the tiles the grid covers: nqt - 1 .. nqt - grid_tiles
    const dim3 grid(8 * xcd_slots(a.BH, p.grid_tiles) * col_parts * p.splits);
    // rows = (K2, V2), streamed = (K1, U): dQ, dK2, dV2
    p.row_k = (const E*)a.k2; p.row_v = (const E*)a.v2;
    p.st_k = (const E*)a.k1; p.st_v = u; p.st_kt = k1t; p.st_vt = ut;
    p.at_row_k = a.at_k2; p.at_row_v = a.at_v2; p.at_st_k = a.at_k1; p.at_st_v = at_u;
    p.acc_k = dk2acc; p.acc_v = dv2acc; p.bit_k = kPoisonDK2; p.bit_v = kPoisonDV2;
    p.wa = a.k1_window; p.wb = a.k2_window; p.lab = a.kk_left; p.rab = a.kk_right;
    hipError_t launch_error = hipSuccess;
    auto launch_rows = [&](bool with_dq) {
        if constexpr (D == 64) {
            if (fuse_tile0) {  // the first launch takes tile 0 along
                auto fused = with_dq ? tdp_bwd_rows_tile0_kernel<E, 64, true, SV> : tdp_bwd_rows_tile0_kernel<E, 64, false, SV>;
                launch_error = ensure_dynamic_smem(reinterpret_cast<const void*>(fused), std::max(smem, f32_bwd_smem<64>()));
                if (launch_error != hipSuccess) return;
                const int t0_x = 8 * xcd_slots(a.BH, 1);
                const int t0_first = tiles < 1024 ? 1 : 0;
                hipLaunchKernelGGL(fused, dim3(grid.x + t0_x * 2 * t0_rounds), dim3(512), std::max(smem, f32_bwd_smem<64>()),
                                   st, p, t0_r0, t0_r1, t0_roles, (int)grid.x, t0_x, t0_first);
                fuse_tile0 = false;
                return;
            }
        }
        hipLaunchKernelGGL(with_dq ? kern_dq : kern_nodq, grid, dim3(nthreads), smem, st, p);
    };
    // a launch whose gradients the caller does not want (null outputs) is skipped
    if (tiles_here > 0 && want_q) launch_rows(true);
    else if (tiles_here > 0 && want_k2) launch_rows(false);
    // rows = (K1, U), streamed = (K2, V2): dK1, dU
    p.row_k = (const E*)a.k1; p.row_v = u;
    p.st_k = (const E*)a.k2; p.st_v = (const E*)a.v2; p.st_kt = k2t; p.st_vt = v2t;
    p.at_row_k = a.at_k1; p.at_row_v = at_u; p.at_st_k = a.at_k2; p.at_st_v = a.at_v2;
    p.acc_k = dk1acc; p.acc_v = duacc; p.bit_k = kPoisonDK1; p.bit_v = kPoisonDU;
    p.wa = a.k2_window; p.wb = a.k1_window; p.lab = a.kk_right; p.rab = a.kk_left;  // the mask with j and k exchanged
    if (tiles_here > 0 && want_k1) launch_rows(false);
    if (launch_error != hipSuccess) return launch_error;

    const size_t n = (size_t)a.BH * a.T * D;
    size_t gridf = (n + 255) / 256;
    if (gridf > 4096) gridf = 4096;
    hipLaunchKernelGGL(bwd_finish_kernel<E>, dim3((unsigned)gridf), dim3(256), 0, st, (const float*)dk1acc,
                       (const float*)duacc, (const float*)dk2acc, (const float*)dv2acc, (const float*)dqacc, a.alpha,
                       (E*)a.dq, (const E*)a.v1, (E*)a.dk1, (E*)a.dv1, (E*)a.dk2, (E*)a.dv2, n,
                       a.deterministic ? 1 : 0,
                       (first_in_f32 && !all_in_f32 && !dqacc) ? (const float*)(ws + l.dq0acc) : nullptr, a.T, D,
                       p.scale_parts, p.poison, p.H, SV ? a.at_v1 : dense_at(1, a.T, D));
    return hipGetLastError();
}

size_t mfma_tdp_bwd_workspace(int BH, int T, int D, bool deterministic) {
    return bwd_layout(BH, T, D, deterministic).total;
}
bool mfma_tdp_bwd_supported(int D, int dtype_is_16bit) { return dtype_is_16bit && (D == 32 || D == 64 || D == 128); }

template <bool SV>
static hipError_t bwd_by_shape(const MfmaBwdArgs& a, hipStream_t st) {
    if (a.D == 32) return a.is_bf16 ? launch_bwd<__bf16, 32, SV>(a, st) : launch_bwd<_Float16, 32, SV>(a, st);
    if (a.D == 64) return a.is_bf16 ? launch_bwd<__bf16, 64, SV>(a, st) : launch_bwd<_Float16, 64, SV>(a, st);
    if (a.D == 128) return a.is_bf16 ? launch_bwd<__bf16, 128, SV>(a, st) : launch_bwd<_Float16, 128, SV>(a, st);
    return hipErrorInvalidValue;
}
hipError_t mfma_tdp_bwd(const MfmaBwdArgs& a, hipStream_t st) {
    return a.H > 0 ? bwd_by_shape<true>(a, st) : bwd_by_shape<false>(a, st);
}

}  // namespace tritt
