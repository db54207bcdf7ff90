// Triple-dot-product trittention backward on MFMA: the general form of the rows kernel (included by
// tdp_bwd_mfma.hip after BwdParams).  It serves head dimensions 32 and 128 and, for head dimensions
// 64 and 128, windowed causal masks (WIN): rounds and steps then cover the band only, and a key outside the
// window of its (q, k) is masked like one past the causal bound.
//
// Same decomposition as tdp_bwd_rows_kernel (rows = one K2/V2 row k per wave and round, K1 / U
// streamed over j, the columns of every tile = 32 queries).  The accumulators Yq / Tv of all 128
// gradient columns are 128 registers, so there are two shapes:
// For D = 128:
//  * NW = 4 waves, NCOL = 128: one wave per SIMD with the whole 512-entry register file; a
//    tile-step (32 keys) is 18 + 16 MFMAs;
//  * NW = 8 waves, NCOL = 64: two waves per SIMD, a workgroup produces one half of the gradient
//    columns (blockIdx carries the half) and both halves recompute S and dP, which still
//    contract over all 128: 18 + 8 MFMAs per tile-step and half.
// -LSE2[q] and -Delta[q] enter S and dP through one extra k-step (A = ones_operand, B =
// offset_operand) instead of two resident 16-register C tiles.  Stages are 32 keys: K1 and U rows
// as 64 x 64 tiles (tile row = 32 * (d / 64) + key, the swizzle of direct_lds.hpp), K1^T and U^T
// of the workgroup's columns as compact [NCOL d][32 keys] tiles; three buffers, fetched
// direct-to-LDS two steps ahead, one workgroup barrier per step.  D = 64 (WIN only; the full-window
// case has its own kernel): NW = 8, NCOL = 64, the row tiles have 32 rows.  D = 32: NW = 8,
// NCOL = 32, the row tiles have 32 rows of 64 bytes (swizzled like the transposed tiles).
#pragma once

namespace tritt {

// An extra k-step whose A operand is `ones_operand` (1 in k-slots 0..2 of every row) and whose B
// operand is `offset_operand(x)` (the three 16-bit pieces of -x in the same slots of the lane's
// column) adds -x to the fp32 accumulator to ~24 bits.
template <typename E>
__device__ __forceinline__ typename Mma<E>::v8 ones_operand(int g) {
    typename Mma<E>::v8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (E)((g == 0 && e < 3) ? 1.0f : 0.0f);
    return r;
}
template <typename E>
__device__ __forceinline__ typename Mma<E>::v8 offset_operand(float x, int g) {
    const float neg = -x;
    const E hi = (E)neg;
    const float r1 = neg - (float)hi;
    const E mid = (E)r1;
    const E lo = (E)(r1 - (float)mid);
    typename Mma<E>::v8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (E)0.0f;
    if (g == 0) {
        r[0] = hi;
        r[1] = mid;
        r[2] = lo;
    }
    return r;
}

// chunk swizzle of the compact transposed tiles: rows are 64 bytes, so rows r, r+4, r+8, r+12
// share banks; 16-byte chunk c of row r sits at position c ^ swz_t(r)
__device__ __forceinline__ constexpr int swz_t(int r) { return (r >> 2) & 3; }

constexpr int bwdg_stage_bytes(int d, int ncol) { return 2 * d * 64 + 2 * ncol * 64; }
// rows of a round buffer: the round's NW rows, or what one 1 KB load brings in if that is more
constexpr int bwdg_round_rows(int d, int nw) { return nw > 512 / d ? nw : 512 / d; }
constexpr size_t bwdg_smem(int d, int nw, int ncol, bool with_dq) {
    return 3 * (size_t)bwdg_stage_bytes(d, ncol)               // stage buffers
           + 2 * (2 * bwdg_round_rows(d, nw) * d * 2)           // K2 / V2 rows of two rounds
           + (ncol == 64 ? 2 * (32 * (d + 4) * 4) : 2 * (32 * (d + 8) * 2))  // Q and dO tiles (64 columns: fp32)
           + (with_dq ? (nw / 2) * (32 * ncol * 4) : 0)         // dQ slices (one per pair of waves)
           + (ncol == 64 ? 2 * (2 * 64 * 16 * 2) : 0);          // Q and dO in accumulator layout (NCOL = 64)
}

// SPLIT: the B operands of the score products, alpha log2e Q (.) K2[k] and dO (.) V2[k], are kept as hi + lo pairs
// of 16-bit numbers (16 mantissa bits together; the streamed K1 / U operands are exact), two MFMAs per k-step: S
// and dP then carry fp32 accumulation error only, and dS = P (dP - Delta) no longer cancels numbers that carry
// 16-bit operand rounding.
// SV: the caller's tensors are strided views (BwdParams::at_*); otherwise everything is dense.
template <typename E, int D, bool WITH_DQ, int NW, int NCOL, bool WIN, bool SPLIT = false, bool SV = false>
__global__ __launch_bounds__(64 * NW) void tdp_bwd_rows_general_kernel(BwdParams<E> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = NCOL / 32, DH = NCOL, BQ = 32, NTH = 64 * NW;
    constexpr int LDK = D + 8;
    constexpr int RB = D / 16;               // 1 KB blocks of a row-major stage tile (32 keys x D)
    constexpr int NBLK = 2 * RB + NCOL / 8;  // blocks of a stage: K1 rows, U rows, NCOL/16 + NCOL/16 transposed
    constexpr int NBUF = 3, LW = NBLK / NW;  // stage buffers; direct loads per wave per stage
    constexpr int STAGE = bwdg_stage_bytes(D, NCOL) / 2;  // elements
    constexpr bool EPI_TILES = NCOL == 64;   // Q / dO kept a second time in accumulator layout
    constexpr int RW = D < 64 ? D : 64;      // elements of a row-major tile row (D = 128: two rows per key)
    constexpr int CPR = RW / 8, RPB = 64 / CPR;  // 16-byte chunks per tile row, tile rows per 1 KB block
    constexpr int RR = bwdg_round_rows(D, NW);   // rows of a round buffer
    static_assert(D == 32 || D == 64 || D == 128, "head dimension");
    static_assert((NW == 8 && NCOL == 64 && D >= 64) || (D == 128 && NW == 4 && NCOL == 128) ||
                  (D == 32 && NW == 8 && NCOL == 32), "workgroup shapes");
    static_assert(NBLK % NW == 0, "whole blocks per wave");
    static_assert(!SPLIT || D <= 64, "split operands: the lo halves of a D = 128 round do not fit the register file");

    extern __shared__ __align__(16) char smem[];
    E* sStage = reinterpret_cast<E*>(smem);  // [NBUF][K1 rows 4096 | U rows 4096 | K1^T 2048 | U^T 2048]
    E* sKr = sStage + NBUF * STAGE;          // [2][RR][D]
    E* sVr = sKr + 2 * RR * D;
    // Q and dO tiles for the operand build.  64-column shapes (where LDS has the room): Q * alpha*log2(e) and dO in
    // fp32, so a product is one conversion and one multiply and S is rounded exactly as the forward rounded it.
    constexpr bool QF = NCOL == 64;
    constexpr int LDQ = D + 4, QT_BYTES = QF ? BQ * LDQ * 4 : BQ * LDK * 2;
    char* qtiles = reinterpret_cast<char*>(sVr + 2 * RR * D);
    E* sQb = reinterpret_cast<E*>(qtiles);              // [BQ][LDK]   (!QF)
    E* sOb = reinterpret_cast<E*>(qtiles + QT_BYTES);
    [[maybe_unused]] float* sQf = reinterpret_cast<float*>(qtiles);  // [BQ][LDQ]   (QF)
    [[maybe_unused]] float* sOf = reinterpret_cast<float*>(qtiles + QT_BYTES);
    float* sDQall = reinterpret_cast<float*>(qtiles + 2 * QT_BYTES);  // [NW/2][BQ * DH], accumulator layout (WITH_DQ)
    float* sDQ = sDQall + (wave_of(threadIdx.x) >> 1) * (BQ * DH);
    E* sQe = reinterpret_cast<E*>(sDQall + (WITH_DQ ? (NW / 2) * (BQ * DH) : 0));  // [DT][64][16] (EPI_TILES)
    E* sOe = sQe + DT * 64 * 16;

    const int xcd = blockIdx.x & 7;
    int slot = blockIdx.x >> 3;
    int c0 = 0;  // first gradient column of this workgroup
    if constexpr (NCOL < D) {
        c0 = (slot & 1) * DH;
        slot >>= 1;
    }
    const int split = slot % p.splits;  // which share of the tile's rows (rounds) this workgroup walks
    slot /= p.splits;
    int bh, order;
    if (!xcd_tile(p.BH, p.grid_tiles, slot, xcd, bh, order)) return;
    const int qt = p.nqt - 1 - order;  // heaviest query tiles first

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D, tbase = (size_t)bh * D * p.Tp;
    const float fscale = acc_scale(p, bh);
    const E* __restrict__ K2 = slice_of<SV, D>(p.row_k, p.at_row_k, bh, p.H, T);
    const E* __restrict__ V2 = slice_of<SV, D>(p.row_v, p.at_row_v, bh, p.H, T);
    const E* __restrict__ Qs = slice_of<SV, D>(p.q, p.at_q, bh, p.H, T);
    const E* __restrict__ Os = slice_of<SV, D>(p.d_o, p.at_do, bh, p.H, T);
    // row pitches in elements
    const unsigned pK2 = pitch_of<SV, D>(p.at_row_k), pV2 = pitch_of<SV, D>(p.at_row_v), pQ = pitch_of<SV, D>(p.at_q),
                   pO = pitch_of<SV, D>(p.at_do), pSK = pitch_of<SV, D>(p.at_st_k), pSV = pitch_of<SV, D>(p.at_st_v);

    const int q0 = qt * BQ;
    const int qlast = min(T - 1, q0 + BQ - 1);
    const int jend = p.causal ? qlast : T - 1;
    const int jfull = p.causal ? q0 : T - 1;
    const int nsteps = jend / 32 + 1, nrounds = jend / NW + 1;
    // WIN, with a = streamed index (j), b = row index (k):  (q, a, b) takes part iff a, b <= q,
    // q - a <= wa, q - b <= wb, b - a <= lab, a - b <= rab.  Rows below b_first are outside the band
    // of every query here; a round's sweep over a covers step_lo(m) .. step_hi(m) (never empty).
    const bool banded = WIN && p.causal;
    const int m_first = banded ? max(0, max(q0 - p.wb, q0 - p.wa - p.rab)) / NW : 0;
    auto step_lo = [&](int m) { return banded ? max(0, max(q0 - p.wa, m * NW - p.lab)) / 32 : 0; };
    auto step_hi = [&](int m) { return banded ? min(jend, m * NW + NW - 1 + p.rab) / 32 : nsteps - 1; };
    // this workgroup's rounds
    const int per_split = (nrounds - m_first + p.splits - 1) / p.splits;
    const int m_lo = m_first + split * per_split, m_hi = min(nrounds, m_lo + per_split);
    if (m_lo >= m_hi) return;  // fewer rounds than shares (uniform over the workgroup, before any barrier)
    const int q = q0 + n;
    const bool q_ok = q < T;
    const int jq = p.causal ? min(q, T - 1) : T - 1;
    const float scale_log2 = p.alpha * kLog2e;

    // ---- stage loader: NBLK blocks of 1 KB, wave w fetches blocks LW w .. LW w + LW - 1
    //   RB blocks of K1 rows, RB of U rows (tile rows 8b .. 8b+7), then NCOL/16 blocks of K1^T and as many
    //   of U^T (16 d-rows each)
    const E* gsrc[LW];
    unsigned goff[LW];     // per-lane byte offset at key 0
    unsigned gstep[LW];    // bytes per key
    int rowkey[LW];        // row-major blocks: key offset of this lane's row inside the stage; else -1
    unsigned rowrest[LW];  // row-major blocks: byte offset inside the row
#pragma unroll
    for (int c = 0; c < LW; ++c) {
        const int b = wave * LW + c;
        if (b < 2 * RB) {
            const int R = (b % RB) * RPB + lane / CPR, hh = R >> 5, r = R & 31;
            const int chunk = (lane % CPR) ^ (D == 32 ? swz_t(r) : swz_perm(r));
            gsrc[c] = uniform_ptr(b < RB ? slice_of<SV, D>(p.st_k, p.at_st_k, bh, p.H, T)
                                         : slice_of<SV, D>(p.st_v, p.at_st_v, bh, p.H, T));
            rowkey[c] = r;
            rowrest[c] = (unsigned)(hh * 64 + chunk * 8) * 2;
            gstep[c] = (b < RB ? pSK : pSV) * 2;
            goff[c] = (unsigned)r * gstep[c] + rowrest[c];
        } else {
            const int dl = ((b - 2 * RB) % (NCOL / 16)) * 16 + (lane >> 2);
            const int chunk = (lane & 3) ^ swz_t(dl);
            gsrc[c] = uniform_ptr((b < 2 * RB + NCOL / 16 ? p.st_kt : p.st_vt) + tbase);
            rowkey[c] = -1;
            rowrest[c] = 0;
            goff[c] = ((unsigned)(c0 + dl) * p.Tp + chunk * 8) * 2;
            gstep[c] = 2;
        }
    }
    auto issue_stage = [&](int st, int buf) {
        const int jb = st * 32;
        char* dst = reinterpret_cast<char*>(sStage + buf * STAGE) + wave * LW * 1024;
        const bool ragged = jb + 31 > T - 1;  // row-major rows past the end of the sequence: clamp
#pragma unroll
        for (int c = 0; c < LW; ++c) {
            unsigned off = goff[c] + (unsigned)jb * gstep[c];
            if (ragged && rowkey[c] >= 0) off = (unsigned)min(jb + rowkey[c], T - 1) * gstep[c] + rowrest[c];
            direct_load_16(gsrc[c], off, dst + c * 1024);
        }
    };
    // the round's K2 / V2 rows NW m .. NW m + NW - 1: one load moves 1 KB = RPL rows
    auto issue_round = [&](int m, int buf) {
        constexpr int RPL = 512 / D, LPR = D / 8;    // rows per load, lanes per row
        constexpr int LR = NW > RPL ? NW / RPL : 1;  // loads per tensor (D = 32: one load brings 16 rows, 8 are used)
        static_assert(2 * LR <= NW, "round loader");
        if (wave < 2 * LR) {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int part = wave % LR;
            const bool second = wave >= LR;
            const unsigned off = (unsigned)min(m * NW + part * RPL + ln / LPR, T - 1) * ((second ? pV2 : pK2) * 2) + (ln % LPR) * 16;
            direct_load_16(uniform_ptr(second ? V2 : K2), off, (second ? sVr : sKr) + buf * RR * D + part * RPL * D);
        }
    };

    // ---- prologue
    for (int idx = tid; idx < BQ * D; idx += NTH) {
        const int r = idx / D, d = idx % D;
        const unsigned row = (unsigned)min(q0 + r, T - 1);
        const E qv = Qs[(size_t)row * pQ + d], ov = Os[(size_t)row * pO + d];
        if constexpr (QF) {
            sQf[r * LDQ + d] = (float)qv * scale_log2;
            sOf[r * LDQ + d] = (float)ov;
        } else {
            sQb[r * LDK + d] = qv;
            sOb[r * LDK + d] = ov;
        }
    }
    if constexpr (EPI_TILES) {
        for (int idx = tid; idx < DT * 64 * 16; idx += NTH) {
            const int i = idx & 15, ln = (idx >> 4) & 63, dt = idx >> 10;
            const unsigned row = (unsigned)min(q0 + c_row(ln >> 5, i), T - 1);
            sQe[idx] = Qs[(size_t)row * pQ + c0 + dt * 32 + (ln & 31)];
            sOe[idx] = Os[(size_t)row * pO + c0 + dt * 32 + (ln & 31)];
        }
    }
    if constexpr (WITH_DQ) {
        for (int idx = tid; idx < (NW / 2) * BQ * DH; idx += NTH) sDQall[idx] = 0.f;
    }
    // (round, step) of the stage fetched next: the sequence the main loop walks, wrapping to the first
    // round after the last (those fetches are never used)
    int m_ahead = m_lo, st_ahead = step_lo(m_lo);
    auto advance = [&]() {
        if (st_ahead < step_hi(m_ahead)) {
            ++st_ahead;
        } else {
            m_ahead = m_ahead + 1 < m_hi ? m_ahead + 1 : m_lo;
            st_ahead = step_lo(m_ahead);
        }
    };
    issue_round(m_lo, m_lo & 1);
    issue_stage(st_ahead, 0);
    advance();
    issue_stage(st_ahead, 1);
    advance();
    int gstage = 0;

    const float lse2 = q_ok ? p.lse[(size_t)bh * T + q] * kLog2e : 3.0e4f;
    const float delta = q_ok ? p.delta[(size_t)bh * T + q] : 0.f;
    const v8 a_ones = ones_operand<E>(g);
    const v8 b_lse = offset_operand<E>(lse2, g), b_delta = offset_operand<E>(delta, g);
    const int krow_off = key_of_row(n);
    const int fperm = D == 32 ? swz_t(krow_off) : swz_perm(krow_off);

    // STAG (the split-operand kernel under full windows, where a step is long enough for it to pay: 17.2 -> 16.9 ms
    // at B=4 H=8 T=1024; the windowed and the D = 32 instantiations measured 1-8 % slower with it): the two waves
    // of a SIMD (w and w + 4) run half a step apart, as in tdp_bwd_rows_kernel.  The barrier of step g then stands
    // for "stage g + 1 has landed for every wave, every wave is done with stage g - 1"; the first wave of a SIMD
    // crosses it at the top of its step, the second after its score products, and a wave's priority is low over
    // its score products and high over the rest of the step.
    constexpr bool STAG = SPLIT && !WIN && D == 64 && NW == 8;
    [[maybe_unused]] const bool late = STAG && ((wave >> 2) & 1);
    if constexpr (STAG) barrier_keep_loads<LW>();  // stage 0 and the first round's rows have landed for every wave
    for (int m = m_lo; m < m_hi; ++m) {
        const int mb = m & 1;
        const int k = m * NW + wave;
        const int st_first = step_lo(m), st_last = step_hi(m);
        // WIN: this lane's window of streamed keys for (q, k); empty if k itself is outside the band of q
        [[maybe_unused]] int wlo = 0, whi = -1;
        if constexpr (WIN) {
            if (k <= jq && (!banded || q <= k + p.wb)) {
                wlo = banded ? max(q - p.wa, k - p.lab) : 0;
                whi = banded ? min(jq, k + p.rab) : jq;
            }
        }

        v8 bq[KS], bg[KS];
        [[maybe_unused]] v8 bql[SPLIT ? KS : 1], bgl[SPLIT ? KS : 1];
        bool built = false;
        f32x16 accQ[DT], accT[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                accQ[dt][i] = 0.f;
                accT[dt][i] = 0.f;
            }

        for (int st = st_first; st <= st_last; ++st, ++gstage) {
            // this wave's part of stage gstage (and, at a round's first step, its part of the round's
            // rows) has landed; after the barrier that holds for every wave's part, and every wave is
            // done with the buffer the next fetch overwrites
            auto stage_barrier = [&]() {
                if constexpr (STAG) barrier_keep_loads<0>();
                else barrier_keep_loads<LW>();
                if (st == st_first && m + 1 < m_hi) issue_round(m + 1, mb ^ 1);  // older than the stage loads
                issue_stage(st_ahead, (gstage + 2) % NBUF);
                advance();
            };
            if (!late) stage_barrier();
            if (!built) {
                // B operands of the score products of this round: alpha log2e Q (.) K2[k] and dO (.) V2[k]
                built = true;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int off = ks * 16 + g * 8;
                    const v8 kv = *reinterpret_cast<const v8*>(sKr + (mb * RR + wave) * D + off);
                    const v8 vv = *reinterpret_cast<const v8*>(sVr + (mb * RR + wave) * D + off);
                    float qf[8], df[8];
                    if constexpr (QF) {
                        const float4 qa = *reinterpret_cast<const float4*>(sQf + n * LDQ + off);
                        const float4 qb = *reinterpret_cast<const float4*>(sQf + n * LDQ + off + 4);
                        const float4 da = *reinterpret_cast<const float4*>(sOf + n * LDQ + off);
                        const float4 db = *reinterpret_cast<const float4*>(sOf + n * LDQ + off + 4);
                        qf[0] = qa.x; qf[1] = qa.y; qf[2] = qa.z; qf[3] = qa.w; qf[4] = qb.x; qf[5] = qb.y; qf[6] = qb.z; qf[7] = qb.w;
                        df[0] = da.x; df[1] = da.y; df[2] = da.z; df[3] = da.w; df[4] = db.x; df[5] = db.y; df[6] = db.z; df[7] = db.w;
                    } else {
                        const v8 qv = *reinterpret_cast<const v8*>(sQb + n * LDK + off);
                        const v8 dv = *reinterpret_cast<const v8*>(sOb + n * LDK + off);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            qf[e] = (float)qv[e] * scale_log2;
                            df[e] = (float)dv[e];
                        }
                    }
                    v8 a, b;
                    [[maybe_unused]] v8 al, bl;
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const float a0 = (float)kv[e] * qf[e], a1 = (float)kv[e + 1] * qf[e + 1];
                        const float b0 = (float)vv[e] * df[e], b1 = (float)vv[e + 1] * df[e + 1];
                        const v2 pa = M::pack(a0, a1);
                        const v2 pb = M::pack(b0, b1);
                        a[e] = pa[0]; a[e + 1] = pa[1];
                        b[e] = pb[0]; b[e + 1] = pb[1];
                        if constexpr (SPLIT) {
                            const v2 la = M::pack(a0 - (float)pa[0], a1 - (float)pa[1]);
                            const v2 lb = M::pack(b0 - (float)pb[0], b1 - (float)pb[1]);
                            al[e] = la[0]; al[e + 1] = la[1];
                            bl[e] = lb[0]; bl[e + 1] = lb[1];
                        }
                    }
                    bq[ks] = a;
                    bg[ks] = b;
                    if constexpr (SPLIT) {
                        bql[ks] = al;
                        bgl[ks] = bl;
                    }
                }
            }

            const E* sb = sStage + (gstage % NBUF) * STAGE;
            const E* sK1 = sb;
            const E* sU = sb + D * 32;
            const E* sK1T = sb + 2 * D * 32;
            const E* sUT = sb + 2 * D * 32 + NCOL * 32;
            const int jb = st * 32;
            bool need_mask = (k > jfull) || (jb + 31 > jfull);
            if constexpr (WIN) {
                // inside the band of every query of the tile (q0 .. q0 + 31), for this wave's row k
                if (banded)
                    need_mask = !((k <= q0) && (q0 + 31 <= k + p.wb) && (jb >= max(q0 + 31 - p.wa, k - p.lab)) &&
                                  (jb + 31 <= min(q0, k + p.rab)));
            }

            // row operands in two batches of four k-steps: the second is read under the first products
            // one batch of row operands at a time: the second batch (D = 128) reuses the registers of the first
            // once its products have been issued
            constexpr int KB = KS < 4 ? KS : 4;
            v8 ak[KB], au[KB];
            auto load_rows = [&](int first) {
#pragma unroll
                for (int ks = first; ks < min(first + 4, KS); ++ks) {
                    const int roff = ((ks >> 2) * 32 + krow_off) * RW + ((((ks & 3) * 2 + g) ^ fperm) * 8);
                    ak[ks & 3] = *reinterpret_cast<const v8*>(sK1 + roff);
                    au[ks & 3] = *reinterpret_cast<const v8*>(sU + roff);
                }
            };
            load_rows(0);
            __builtin_amdgcn_sched_barrier(0);
            // S starts from 0, or from -3e4 where (q, j, k) is invalid; element i of a lane is key
            // jb + key_of(0, i) + 8 g.  The extra k-step subtracts LSE2[q] / Delta[q].
            if constexpr (STAG) __builtin_amdgcn_s_setprio(0);
            f32x16 s, dp;
            {
                f32x16 c;
#pragma unroll
                for (int i = 0; i < 16; ++i) c[i] = 0.f;
                dp = M::mma(a_ones, b_delta, c);
                if (need_mask) {
                    if constexpr (WIN) {
                        const int lo = wlo - jb - 8 * g, hi = whi - jb - 8 * g;
#pragma unroll
                        for (int i = 0; i < 16; ++i) c[i] = (key_of(0, i) >= lo && key_of(0, i) <= hi) ? 0.f : -3.0e4f;
                    } else {
                        const int lim = (k <= jq) ? jq - jb - 8 * g : -1;
#pragma unroll
                        for (int i = 0; i < 16; ++i) c[i] = key_of(0, i) <= lim ? 0.f : -3.0e4f;
                    }
                }
                s = M::mma(a_ones, b_lse, c);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < KB; ++ks) {
                s = M::mma(ak[ks], bq[ks], s);
                dp = M::mma(au[ks], bg[ks], dp);
                if constexpr (SPLIT) {
                    s = M::mma(ak[ks], bql[ks], s);
                    dp = M::mma(au[ks], bgl[ks], dp);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (KS > 4) {
                load_rows(4);  // lands under the products just issued
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 4; ks < KS; ++ks) {
                    s = M::mma(ak[ks & 3], bq[ks], s);
                    dp = M::mma(au[ks & 3], bg[ks], dp);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (STAG) {
                if (late) stage_barrier();
                __builtin_amdgcn_sched_barrier(0);
                if (late) __builtin_amdgcn_s_setprio(2);  // one level above the first wave: the two never tie
                else __builtin_amdgcn_s_setprio(1);
            }
            v8 bt[DT][2], bk[DT][2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int dl = dt * 32 + n;
                    const int toff = dl * 32 + (((h * 2 + g) ^ swz_t(dl)) * 8);
                    bt[dt][h] = *reinterpret_cast<const v8*>(sUT + toff);
                    bk[dt][h] = *reinterpret_cast<const v8*>(sK1T + toff);
                }
            __builtin_amdgcn_sched_barrier(0);
            v8 pa[2], da[2];
            // SPLIT, in the launch that produces dQ: dS as a hi + lo pair too.  dQ[q] sums dS K1 (.) K2 over the (j, k)
            // of ONE softmax row, terms of both signs that cancel when the row is close to one-hot, so the 8-bit
            // rounding of a single 16-bit operand shows there (measured: 1.4 x the tolerance at scores spanning
            // hundreds, 0.2 x with the pair).  The row gradients sum over many queries and P feeds sums of one
            // sign: neither needs it (the launch without dQ stays at one operand).
            constexpr bool SPLIT_DS = SPLIT && WITH_DQ;
            [[maybe_unused]] v8 dal[SPLIT_DS ? 2 : 1];
            auto softmax_pair = [&](int r) {  // register pair r (0..7): P = exp2(S), dS = P dP, packed
                const int h = r >> 2, e = 2 * (r & 3), i = h * 8 + e;
                const float p0 = fast_exp2(s[i]), p1 = fast_exp2(s[i + 1]);
                const v2 pp = M::pack(p0, p1);
                const float d0 = p0 * dp[i], d1 = p1 * dp[i + 1];
                const v2 dd = M::pack(d0, d1);
                pa[h][e] = pp[0]; pa[h][e + 1] = pp[1];
                da[h][e] = dd[0]; da[h][e + 1] = dd[1];
                if constexpr (SPLIT_DS) {
                    const v2 dl = M::pack(d0 - (float)dd[0], d1 - (float)dd[1]);
                    dal[h][e] = dl[0]; dal[h][e + 1] = dl[1];
                }
            };
#pragma unroll
            for (int r = 0; r < 4; ++r) softmax_pair(r);
            __builtin_amdgcn_sched_barrier(0);
            // gradient product r of half h (0 .. 2 DT - 1): even -> Tv += P U, odd -> Yq += dS K1
            auto grad = [&](int h, int r) {
                if ((r & 1) == 0) {
                    accT[r >> 1] = M::mma(pa[h], bt[r >> 1][h], accT[r >> 1]);
                } else {
                    accQ[r >> 1] = M::mma(da[h], bk[r >> 1][h], accQ[r >> 1]);
                    if constexpr (SPLIT_DS) accQ[r >> 1] = M::mma(dal[h], bk[r >> 1][h], accQ[r >> 1]);
                }
            };
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (r < 2 * DT) grad(0, r);
                __builtin_amdgcn_sched_barrier(0);
                softmax_pair(4 + r);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 4; r < 2 * DT; ++r) grad(0, r);
#pragma unroll
            for (int r = 0; r < 2 * DT; ++r) grad(1, r);
            __builtin_amdgcn_sched_barrier(0);
        }

        // ---- round epilogue (rows of the accumulators = the 32 queries, column = c0 + 32 dt + n)
        // registers 8 part .. 8 part + 7 of every accumulator tile: slice += Yq (.) K2[k]
        [[maybe_unused]] auto add_dq = [&](auto part_c) {
            constexpr int part = decltype(part_c)::value;  // compile time: a run-time choice of registers would be
                                                           // indexed through M0, which the direct loads own
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const float kd = (float)sKr[(mb * RR + wave) * D + c0 + dt * 32 + n];
#pragma unroll
                for (int i4 = 2 * part; i4 < 2 * part + 2; ++i4) {
                    float4* slot4 = reinterpret_cast<float4*>(sDQ + ((dt * 4 + i4) * 64 + lane) * 4);
                    float4 v = *slot4;
                    v.x += accQ[dt][i4 * 4] * kd; v.y += accQ[dt][i4 * 4 + 1] * kd;
                    v.z += accQ[dt][i4 * 4 + 2] * kd; v.w += accQ[dt][i4 * 4 + 3] * kd;
                    *slot4 = v;
                }
            }
        };
        if (k <= jend) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int d = c0 + dt * 32 + n;
                float sk = 0.f, sv = 0.f;
                if constexpr (EPI_TILES) {
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
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        sk += accQ[dt][i] * (float)sQb[c_row(g, i) * LDK + d];
                        sv += accT[dt][i] * (float)sOb[c_row(g, i) * LDK + d];
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
        // the two waves of a pair add their tiles to the pair's slice half and half: before the barrier the even wave
        // its first eight registers per tile and the odd wave its last eight, after it the other halves (one wave
        // before and one after would put two chains of dependent LDS round trips of twice the length on the
        // workgroup's path)
        if constexpr (WITH_DQ) {
            if (k <= jend) {
                if (wave & 1) add_dq(std::integral_constant<int, 1>{});
                else add_dq(std::integral_constant<int, 0>{});
            }
        }
        // all waves are done with this round's K2/V2 rows; the next round's have landed (they are older
        // than the stage loads kept in flight)
        if constexpr (STAG) barrier_keep_loads<LW>();  // the round's load is older than the one stage in flight
        else barrier_keep_loads<2 * LW>();
        if constexpr (WITH_DQ) {
            if (k <= jend) {
                if (wave & 1) add_dq(std::integral_constant<int, 0>{});
                else add_dq(std::integral_constant<int, 1>{});
            }
        }
    }
    wait_vmcnt<0>();  // the stages fetched ahead land in LDS before the workgroup ends
    __syncthreads();

    if constexpr (WITH_DQ) {
        // dQ: sum the pairs' slices; a thread takes four consecutive accumulator registers (= four consecutive
        // query rows of one column) at a time
#pragma unroll
        for (int t = 0; t < (BQ * DH / 4 + NTH - 1) / NTH; ++t) {
            const int idx4 = t * NTH + tid, slot4 = idx4 >> 6, ln = idx4 & 63;
            if (idx4 >= BQ * DH / 4) break;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int sl = 0; sl < NW / 2; ++sl) {
                const float4 x = *reinterpret_cast<const float4*>(sDQall + sl * (BQ * DH) + idx4 * 4);
                v.x += x.x; v.y += x.y; v.z += x.z; v.w += x.w;
            }
            const int d = c0 + (slot4 >> 2) * 32 + (ln & 31), r0 = c_row(ln >> 5, (slot4 & 3) * 4);
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
}

}  // namespace tritt
