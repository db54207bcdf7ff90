// Triple-dot-product trittention forward on MFMA (gfx950), 16-bit tensors, D = 32, 64 or 128;
// full causal windows or no mask, and (WIN instantiations) windowed causal masks.
//
// Formulation.  For a fixed key-2 row k the scores of query q are an ordinary attention row:
//   s[q,j,k] = (alpha * Q[q] (.) K2[k]) . K1[j]
// so every pair (q,k) is a "virtual query row" with its own online softmax over j and its own
// accumulator  Tv[(q,k), :] = sum_j P U[j, :]   (U = SiLU(V1)).  The rows of one query are
// merged once per k-tile:  O[q] = sum_k w_k * V2[k] (.) Tv[(q,k)],  w_k = exp2(m_qk - M_q).
//
// Work decomposition.  One workgroup = WAVES waves = BQ = WAVES*NT queries of one (batch, head)
// (D=64: 8 waves x 2 queries at 2 waves per SIMD; D=128: 8 waves x 1 query).  A wave owns NT
// queries; a 32x32 MFMA tile is 32 consecutive k (columns) of ONE query, so the causal bound
// j <= q is uniform over a tile and the k-merge stays inside the wave.
// Outer loop: k-tiles of 32.  Inner loop: JS-row stages of K1 and U^T, staged through LDS and
// shared by all waves (double buffered, one barrier per stage).
//
// Per 32-key step and tile:  S^T = K1 * QK2^T  (rows = j, cols = virtual rows).  The common
// (FAST) sweep takes P = exp2(S) with no reference maximum at all and only records whether
// some row left the safe exponent range; if one did, the workgroup repeats that k-tile with the
// CAREFUL sweep: online softmax whose reference maximum is raised only when a score exceeds it
// by more than 2^8 ("lazy" max).  P is packed to 16 bit in the registers it already occupies
// and fed straight back as the A operand of Tv += P * U.
//
// Small grids: the k-tiles of a query tile are dealt out to several workgroups (FwdParams::splits), each
// writes its unnormalised output, reference maximum and row sum, and fwd_merge_kernel joins them.
// Narrow windowed masks take another kernel altogether (tdp_fwd_band.hpp): the whole band of a query
// tile resident in LDS, waves independent after one barrier.
#include <stdlib.h>

#include <type_traits>

#include "kernels.hpp"
#include "mfma.hpp"

namespace tritt {

template <typename E>
struct FwdParams {
    const E *q, *k1, *k2, *v2;
    const E* ut;  // [BH][D][Tp]  SiLU(V1) transposed, zero padded to Tp (multiple of 64)
    // Q, K1, K2, V2 are views of one layout: element (b, h, t, d) at b in_sb + h in_sh + t in_st + d.  The outputs, U^T
    // and the parts are dense.
    long long in_sb, in_sh;
    unsigned in_st;
    int H;
    // MV ("many views") instantiations only: K1, K2 and V2 on layouts of their own (in_* is then Q's)
    TensorAt at_k1, at_k2, at_v2;
    E* o;
    E* o_res;  // SPLIT: the rounding residual of every output element, O(fp32) - O(16 bit), as a second tensor
    float* lse;
    int T, Tp, BH, nqt;
    float scale_log2;
    int causal;
    // windowed instantiation only: (q, j, k) takes part iff j <= q, k <= q, q - j <= wa, q - k <= wb,
    // k - j <= lab, j - k <= rab
    int wa, wb, lab, rab;
    // splits > 1 (small grids): the k-tiles of a query tile are dealt out to `splits` workgroups; each writes
    // its unnormalised output, reference maximum and row sum to part[((bh T + q) splits + s) (D + 2)]
    // (O[D], M, L; M in log2 units, -inf: nothing in this part) and fwd_merge_kernel joins them
    int splits;
    float* part;
};

constexpr float kLazyThreshold = 8.0f;

__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// Smallest row sum the FAST sweep (P = exp2(score), reference 0) accepts.  bf16 has the exponent range of fp32, so
// only a vanished sum is refused.  fp16 loses mantissa bits below 2^-14 and flushes below 2^-24: a row whose sum is
// under 2^-10 was summed from values in that range and is redone with a running maximum.
template <typename E>
__device__ __forceinline__ constexpr float fast_row_sum_floor() {
    return std::is_same<E, _Float16>::value ? 9.765625e-4f : 1e-30f;
}

// MINW (second launch-bounds argument): waves per SIMD the register allocator must leave room for
// WIN: windowed causal masks.  The k-tile and stage loops run over the band only, every step goes
// through the general (per tile, element-wise masked) loop, and the CAREFUL sweep tolerates rows whose
// first valid key comes late.
// MDIAG (NT = 1 only): the stages on the causal diagonal run the interleaved loop too, masked through the C
// operand, instead of the general loop.  Not instantiated: at D = 128 it needs 40 bytes of scratch per lane and
// measures no faster where the diagonal is the largest share of the work (B=1 H=16 bf16: T=512 0.492 ms against
// 0.489 ms with the general loop, T=768 1.334 against 1.323).
// SPLIT: the B operand of the score product, alpha log2e Q[q] (.) K2[k], is a product of two 16-bit numbers and a
// scale: rounded to one 16-bit operand it loses half its bits, and scores that span hundreds then differ from the
// exact ones by more than the softmax can absorb.  SPLIT keeps it as hi + lo (hi = the rounded product, lo = the
// rounded remainder: 16 mantissa bits together) and issues two score MFMAs per k-step, K1 hi and K1 lo.  K1 itself
// is exact (an input), so the scores carry fp32 accumulation error only.  The lo operands live in LDS (one
// kilobyte per tile and k-step, private to the wave).  The output is stored with its rounding residual (o_res), so
// the backward's Delta = rowsum(dO * O) does not inherit the 16-bit rounding of O.  (P as a hi + lo pair in the
// value product was measured as well: no effect on any gradient at scores spanning hundreds, 40 % more time.)
// MV: Q, K1, K2 and V2 each on a layout of its own (FwdParams::at_*) instead of one common layout.
template <typename E, int D, int NT, int WAVES, int MINW, int JS, bool WIN = false, bool MDIAG = false, bool SPLIT = false,
          bool MV = false>
__global__ __launch_bounds__(64 * WAVES, MINW) void tdp_fwd_mfma_kernel(FwdParams<E> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int NTH = 64 * WAVES;
    constexpr int KS = D / 16;   // k-steps of the score product
    constexpr int DT = D / 32;   // 32-wide d tiles of the value product
    constexpr int BQ = WAVES * NT;
    constexpr int LDK = D + 8;   // LDS row stride (elements) of row-major [rows][D] tiles
    constexpr int LDQ = D + 4;   // row stride (floats) of the pre-scaled Q tile
    constexpr int LDU = JS + 8;  // LDS row stride of the U^T stage ([D][JS keys])
    constexpr int K1_CHUNKS = JS * D / 8;      // 16-byte chunks of a K1 stage [JS][D]
    constexpr int STAGE_CHUNKS = 2 * K1_CHUNKS;  // ... followed by the U^T stage [D][JS]
    constexpr int KTILE_CHUNKS = 8 * D;   // K2 [32][D] then V2 [32][D]
    constexpr int CS = (STAGE_CHUNKS + NTH - 1) / NTH, CK = (KTILE_CHUNKS + NTH - 1) / NTH;

    extern __shared__ __align__(16) char smem[];
    E* sK1 = reinterpret_cast<E*>(smem);  // [2][JS][LDK]
    E* sUT = sK1 + 2 * JS * LDK;          // [2][D][LDU]
    E* sK2 = sUT + 2 * D * LDU;           // [2][32][LDK]
    E* sV2 = sK2 + 2 * 32 * LDK;          // [2][32][LDK]
    float* sQ = reinterpret_cast<float*>(sV2 + 2 * 32 * LDK);  // [BQ][LDQ] Q * alpha*log2(e), fp32
    float* sW = sQ + BQ * LDQ;                                  // [WAVES][32] per-wave scratch
    int* sFlag = reinterpret_cast<int*>(sW + WAVES * 32);
    // SPLIT: lo operands of this wave's tiles, [NT][KS][64 lanes][8]
    [[maybe_unused]] E* sLo = reinterpret_cast<E*>(sFlag + 4) + (size_t)wave_index() * (NT * KS * 512);

    // heavy-first, XCD-aware block order: consecutive block ids go to different XCDs, so give
    // every XCD its own set of heads (their K/V stay in that XCD's L2) and hand out the
    // longest query tiles first.
    const int xcd = blockIdx.x & 7;
    int slot = blockIdx.x >> 3;
    const int split = slot % p.splits;
    slot /= p.splits;
    int bh, order;
    if (!xcd_tile(p.BH, p.nqt, slot, xcd, bh, order)) return;
    const int qt = p.nqt - 1 - order;

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it scalar
    const int T = p.T;
    const size_t base = (size_t)bh * T * D;  // of the outputs
    const size_t in_base = (size_t)(bh / p.H) * p.in_sb + (size_t)(bh % p.H) * p.in_sh;
    const unsigned in_st = p.in_st;  // row stride of the inputs, elements; (T - 1) in_st + D fits 32 bits
    const E* __restrict__ Q = p.q + in_base;
    auto slice = [&](const E* t, const TensorAt& at) {
        return MV ? t + (size_t)(bh / p.H) * at.sb + (size_t)(bh % p.H) * at.sh : t + in_base;
    };
    const E* __restrict__ K1 = slice(p.k1, p.at_k1);
    const E* __restrict__ K2 = slice(p.k2, p.at_k2);
    const E* __restrict__ V2 = slice(p.v2, p.at_v2);
    const unsigned st_k1 = MV ? p.at_k1.st : in_st, st_k2 = MV ? p.at_k2.st : in_st, st_v2 = MV ? p.at_v2.st : in_st;
    const E* __restrict__ UT = p.ut + (size_t)bh * D * p.Tp;
    float* sWw = sW + wave * 32;

    const int q0 = qt * BQ;
    const int jend = p.causal ? min(T - 1, q0 + BQ - 1) : T - 1;  // last key any query here needs
    const int nst = jend / JS + 1;
    int nkt = jend / 32 + 1;
    // WIN: the first k-tile any query here can use (k >= q - wb, and some j with q - wa <= j <= k + rab),
    // and per k-tile the stages that hold keys j any (q, k) of it can use
    const bool banded = WIN && p.causal;
    int kt_lo = banded ? max(0, max(q0 - p.wb, q0 - p.wa - p.rab)) / 32 : 0;
    if (p.splits > 1) {  // this workgroup's share of the k-tiles
        const int per = (nkt - kt_lo + p.splits - 1) / p.splits;
        kt_lo += split * per;
        nkt = min(nkt, kt_lo + per);
        if (kt_lo >= nkt) {  // nothing left for this part: say so and leave
            const int q = q0 + (int)(threadIdx.x >> 6) * NT + (int)(threadIdx.x & 63);
            if ((threadIdx.x & 63) < NT && q < p.T)
                p.part[(((size_t)bh * p.T + q) * p.splits + split) * (D + 2) + D] = -INFINITY;
            return;
        }
    }
    auto first_stage = [&](int kt) { return banded ? max(0, max(q0 - p.wa, kt * 32 - p.lab)) / JS : 0; };
    auto last_stage = [&](int kt) { return banded ? min(jend, kt * 32 + 31 + p.rab) / JS : nst - 1; };

    int qrow[NT], jmax[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        qrow[t] = q0 + wave * NT + t;
        jmax[t] = p.causal ? min(qrow[t], T - 1) : T - 1;  // bound on j and on k
    }

    // ---- staging helpers ------------------------------------------------------------------
    // one stage = K1 [JS][D] then U^T [D][JS], 16-byte chunks dealt out to the threads: either one
    // chunk per thread (ra0) or CH from each (ra* from K1, rb* from U^T)
    constexpr int CH = K1_CHUNKS >= NTH ? K1_CHUNKS / NTH : 1;
    static_assert(CS == 1 || K1_CHUNKS % NTH == 0, "stage chunks per thread");
    static_assert(CH <= 2 && CK <= 2, "staging registers are named, not indexed (indexed ones end up in scratch memory)");
    uint4 ra0, ra1, rb0, rb1, rkv0, rkv1;
    auto k1_chunk = [&](int item, int jb) {
        const int r = item / (D / 8), ch = item % (D / 8);
        return reinterpret_cast<const uint4*>(K1 + (size_t)((unsigned)min(jb + r, T - 1) * st_k1) + ch * 8);
    };
    auto ut_chunk = [&](int i2, int jb) {
        const int d = i2 / (JS / 8), cj = i2 % (JS / 8);
        return reinterpret_cast<const uint4*>(UT + (size_t)d * p.Tp + jb + cj * 8);
    };
    auto k1_slot = [&](int item, int buf) {
        const int r = item / (D / 8), ch = item % (D / 8);
        return reinterpret_cast<uint4*>(sK1 + (buf * JS + r) * LDK + ch * 8);
    };
    auto ut_slot = [&](int i2, int buf) {
        const int d = i2 / (JS / 8), cj = i2 % (JS / 8);
        return reinterpret_cast<uint4*>(sUT + (buf * D + d) * LDU + cj * 8);
    };
    auto issue_stage = [&](int st) {
        const int jb = st * JS;
        if constexpr (CS > 1) {
            ra0 = *k1_chunk(tid, jb);
            rb0 = *ut_chunk(tid, jb);
            if constexpr (CH == 2) {
                ra1 = *k1_chunk(tid + NTH, jb);
                rb1 = *ut_chunk(tid + NTH, jb);
            }
        } else {
            if (tid < K1_CHUNKS) ra0 = *k1_chunk(tid, jb);
            else if (tid < STAGE_CHUNKS) ra0 = *ut_chunk(tid - K1_CHUNKS, jb);
        }
    };
    auto commit_stage = [&](int buf) {
        if constexpr (CS > 1) {
            *k1_slot(tid, buf) = ra0;
            *ut_slot(tid, buf) = rb0;
            if constexpr (CH == 2) {
                *k1_slot(tid + NTH, buf) = ra1;
                *ut_slot(tid + NTH, buf) = rb1;
            }
        } else {
            if (tid < K1_CHUNKS) *k1_slot(tid, buf) = ra0;
            else if (tid < STAGE_CHUNKS) *ut_slot(tid - K1_CHUNKS, buf) = ra0;
        }
    };
    // K2 [32][D] then V2 [32][D]: the guard is compiled in only when the chunks do not divide evenly
    // (a guarded, indexed register array ends up in scratch memory)
    constexpr bool KT_EVEN = KTILE_CHUNKS % NTH == 0;
    auto kt_src = [&](int item, int kt) {
        const int which = item / (4 * D), rem = item % (4 * D);
        const int r = rem / (D / 8), ch = rem % (D / 8);
        return reinterpret_cast<const uint4*>((which ? V2 : K2) + (size_t)((unsigned)min(kt * 32 + r, T - 1) * (which ? st_v2 : st_k2)) + ch * 8);
    };
    auto kt_dst = [&](int item, int buf) {
        const int which = item / (4 * D), rem = item % (4 * D);
        const int r = rem / (D / 8), ch = rem % (D / 8);
        return reinterpret_cast<uint4*>((which ? sV2 : sK2) + (buf * 32 + r) * LDK + ch * 8);
    };
    auto issue_ktile = [&](int kt) {
        if (KT_EVEN || tid < KTILE_CHUNKS) rkv0 = *kt_src(tid, kt);
        if constexpr (CK == 2) {
            if (KT_EVEN || tid + NTH < KTILE_CHUNKS) rkv1 = *kt_src(tid + NTH, kt);
        }
    };
    auto commit_ktile = [&](int buf) {
        if (KT_EVEN || tid < KTILE_CHUNKS) *kt_dst(tid, buf) = rkv0;
        if constexpr (CK == 2) {
            if (KT_EVEN || tid + NTH < KTILE_CHUNKS) *kt_dst(tid + NTH, buf) = rkv1;
        }
    };
    // broadcast a per-virtual-row scalar (held by lane n) to the C/D layout (rows in registers):
    // out[i] = value of row c_row(g, i).  Goes through this wave's own LDS scratch.
    auto rows_of = [&](float v, float (&out)[16]) {
        if (g == 0) sWw[n] = v;
        __builtin_amdgcn_wave_barrier();  // same wave, same LDS queue: program order is enough
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float4 f4 = *reinterpret_cast<const float4*>(sWw + 8 * b + 4 * g);
            out[4 * b] = f4.x; out[4 * b + 1] = f4.y; out[4 * b + 2] = f4.z; out[4 * b + 3] = f4.w;
        }
        __builtin_amdgcn_wave_barrier();
    };

    // ---- prologue: Q tile, first k-tile, first stage ------------------------------------------
    for (int idx = tid; idx < BQ * D; idx += NTH) {
        const int r = idx / D, d = idx % D;
        sQ[r * LDQ + d] = (float)Q[(size_t)((unsigned)min(q0 + r, T - 1) * in_st) + d] * p.scale_log2;
    }
    if (tid < 2) sFlag[tid] = 0;  // two flags, used by alternate k-tiles
    issue_ktile(kt_lo);
    issue_stage(first_stage(kt_lo));
    commit_ktile(0);
    commit_stage(0);
    __syncthreads();

    float Mrun[NT], Lrun[NT], Orun[NT][DT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        Mrun[t] = -INFINITY;
        Lrun[t] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) Orun[t][dt] = 0.f;
    }

    const int krow_off = key_of_row(n);  // K1 row (within a 32-key step) this lane feeds to the MFMA

    int gstage = 0;  // running stage counter (buffer = gstage & 1)
    [[maybe_unused]] bool plain = true;  // every k-tile so far was merged with reference 0 (see the merge below)
    for (int kt = kt_lo; kt < nkt; ++kt) {
        const int kb = (kt - kt_lo) & 1;
        const int st_lo = first_stage(kt), st_hi = last_stage(kt);
        // the stage fetched after the last one: the next k-tile starts from it (or a repeat of this one)
        const int st_next = kt + 1 < nkt ? first_stage(kt + 1) : st_lo;
        // per-lane window of keys j for the virtual row (q, k = 32 kt + n); hi < lo: the row is empty
        [[maybe_unused]] int wlo[NT], whi[NT];
        if constexpr (WIN) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int k = kt * 32 + n, q = qrow[t];
                wlo[t] = banded ? max(q - p.wa, k - p.lab) : 0;
                whi[t] = banded ? min(jmax[t], k + p.rab) : jmax[t];
                if (k > jmax[t] || (banded && q > k + p.wb)) whi[t] = -1;
                if (whi[t] < wlo[t]) { wlo[t] = 0; whi[t] = -1; }
            }
        }

        // B operands: QK2[(q, k), d] = Q[q,d] * K2[k,d] * alpha*log2(e), k = 32*kt + n
        v8 bq[NT][KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const v8 kv = *reinterpret_cast<const v8*>(sK2 + (kb * 32 + n) * LDK + ks * 16 + g * 8);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float* qp = sQ + (wave * NT + t) * LDQ + ks * 16 + g * 8;
                const float4 qa = *reinterpret_cast<const float4*>(qp), qb = *reinterpret_cast<const float4*>(qp + 4);
                const float qf[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
                v8 r;
                [[maybe_unused]] v8 rl;
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float x0 = (float)kv[e] * qf[e], x1 = (float)kv[e + 1] * qf[e + 1];
                    const v2 pr = M::pack(x0, x1);
                    r[e] = pr[0];
                    r[e + 1] = pr[1];
                    if constexpr (SPLIT) {
                        const v2 pl = M::pack(x0 - (float)pr[0], x1 - (float)pr[1]);
                        rl[e] = pl[0];
                        rl[e + 1] = pl[1];
                    }
                }
                bq[t][ks] = r;
                if constexpr (SPLIT) *reinterpret_cast<v8*>(sLo + ((t * KS + ks) * 64 + lane) * 8) = rl;
            }
        }
        // lo operand of tile t, k-step ks (the wave reads back what it wrote: program order is enough)
        [[maybe_unused]] auto lo_of = [&](int t, int ks) {
            return *reinterpret_cast<const v8*>(sLo + ((t * KS + ks) * 64 + lane) * 8);
        };

        f32x16 acc[NT][DT];
        float mref[NT], lsum[NT];

        // One sweep over j for this k-tile.  FAST: P = exp2(s) with the reference left at 0 and no
        // max tracking at all (scores of ordinary inputs are nowhere near the fp32 exponent range);
        // if that over- or underflows, the sweep is repeated once with CAREFUL = true, the usual
        // online softmax with a lazily raised reference maximum.
        auto sweep = [&](auto careful_tag) {
            constexpr bool CAREFUL = decltype(careful_tag)::value;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                mref[t] = 0.f;
                lsum[t] = 0.f;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[t][dt][i] = 0.f;
            }
            int st = st_lo;
            [[maybe_unused]] bool started[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) started[t] = false;
            // the general loop: any mask, any tile validity, FAST or CAREFUL; runs the stages st .. upto - 1
            auto general_until = [&](int upto) {
            for (; st < upto; ++st, ++gstage) {
                const int sb = gstage & 1;
                // the first stage is fetched again after the last one: the next k-tile, or a CAREFUL
                // repeat of this one, starts from it
                const bool more = (st < st_hi) || (kt + 1 < nkt) || !CAREFUL;
                if (more) issue_stage(st < st_hi ? st + 1 : st_next);
                if (st == st_lo && kt + 1 < nkt) issue_ktile(kt + 1);

#pragma unroll
                for (int half = 0; half < JS / 32; ++half) {
                    const int jb = st * JS + half * 32;
                    if (jb > jend) break;
                    const bool first = (jb == 0);
                    const E* k1p = sK1 + (sb * JS + half * 32 + krow_off) * LDK + g * 8;
                    const E* utp = sUT + (sb * D + n) * LDU + half * 32 + g * 8;

#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        if (jb > jmax[t]) continue;  // tile entirely above the causal bound (wave-uniform)
                        bool inside = true;  // WIN: every (j, k) of this step is valid for the query
                        if constexpr (WIN) {
                            if (banded) {
                                const int q = qrow[t], k0 = kt * 32;
                                // no k of the tile, or no j of the step, is inside the band of this query
                                if (k0 > jmax[t] || q > k0 + 31 + p.wb) continue;
                                if (jb > min(jmax[t], k0 + 31 + p.rab) || jb + 31 < max(q - p.wa, k0 - p.lab)) continue;
                                inside = (k0 + 31 <= jmax[t]) && (q <= k0 + p.wb) && (jb >= max(q - p.wa, k0 + 31 - p.lab)) &&
                                         (jb + 31 <= min(jmax[t], k0 + p.rab));
                            } else {
                                inside = jb + 31 <= jmax[t];
                            }
                        }
                        f32x16 s;
#pragma unroll
                        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            const v8 kop = *reinterpret_cast<const v8*>(k1p + ks * 16);
                            s = M::mma(kop, bq[t][ks], s);
                            if constexpr (SPLIT) s = M::mma(kop, lo_of(t, ks), s);
                        }
                        if constexpr (WIN) {
                            if (!inside) {
#pragma unroll
                                for (int i = 0; i < 16; ++i) {
                                    const int j = jb + key_of(g, i);
                                    s[i] = (j >= wlo[t] && j <= whi[t]) ? s[i] : -INFINITY;
                                }
                            }
                        } else if (jb + 31 > jmax[t]) {
#pragma unroll
                            for (int i = 0; i < 16; ++i) s[i] = (jb + key_of(g, i) <= jmax[t]) ? s[i] : -INFINITY;
                        }
                        if constexpr (CAREFUL && WIN) {
                            // as below, but a row may have seen no valid key yet: its reference then sits at
                            // a finite floor, and the reference is assigned, not incremented (floor + step
                            // would round the step away)
                            float mx = fmaxf(s[0], s[1]);
#pragma unroll
                            for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
                            const bool begin = !started[t];
                            started[t] = true;
                            if (begin || __any(mx - mref[t] > kLazyThreshold)) {
                                const float rmax = fmaxf(fmaxf(mx, __shfl_xor(mx, 32, 64)), -1.0e30f);
                                const float newref = begin ? rmax : fmaxf(rmax, mref[t]);
                                const float f = fast_exp2(mref[t] - newref);
                                mref[t] = newref;
                                if (!begin) {
                                    lsum[t] *= f;
                                    float fr[16];
                                    rows_of(f, fr);
#pragma unroll
                                    for (int i = 0; i < 16; ++i)
#pragma unroll
                                        for (int dt = 0; dt < DT; ++dt) acc[t][dt][i] *= fr[i];
                                }
                            }
                        } else if constexpr (CAREFUL) {
                            float mx = fmaxf(s[0], s[1]);
#pragma unroll
                            for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
                            if (first || __any(mx - mref[t] > kLazyThreshold)) {
                                // raise the reference maximum of the rows that need it (rare)
                                const float rmax = fmaxf(mx, __shfl_xor(mx, 32, 64));
                                const float delta = first ? rmax - mref[t] : fmaxf(rmax - mref[t], 0.f);
                                mref[t] += delta;
                                if (!first) {
                                    const float f = fast_exp2(-delta);
                                    lsum[t] *= f;
                                    float fr[16];
                                    rows_of(f, fr);
#pragma unroll
                                    for (int i = 0; i < 16; ++i)
#pragma unroll
                                        for (int dt = 0; dt < DT; ++dt) acc[t][dt][i] *= fr[i];
                                }
                            }
                        }
                        v8 pa[2];
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
#pragma unroll
                            for (int e = 0; e < 8; e += 2) {
                                float x0 = s[h * 8 + e], x1 = s[h * 8 + e + 1];
                                if constexpr (CAREFUL) {
                                    x0 -= mref[t];
                                    x1 -= mref[t];
                                }
                                const v2 pr = M::pack(fast_exp2(x0), fast_exp2(x1));
                                lsum[t] = M::add_pair(pr, lsum[t]);
                                pa[h][e] = pr[0];
                                pa[h][e + 1] = pr[1];
                            }
                        }
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                            for (int h = 0; h < 2; ++h)
                                acc[t][dt] = M::mma(pa[h], *reinterpret_cast<const v8*>(utp + dt * 32 * LDU + h * 16),
                                                    acc[t][dt]);
                        }
                    }
                }

                if (more) commit_stage(sb ^ 1);
                __syncthreads();
            }
            };
            if constexpr (NT == 2 && !CAREFUL) {
                // Stages whose 64 keys lie inside the causal bound of both tiles of this wave: a loop
                // without branches on tile validity, so the accumulators stay in place (no copies
                // at control-flow joins) and the wave itself overlaps matrix and vector work.  The
                // arbiter serves the oldest wave first and all waves of a workgroup reach the same
                // phase together, so overlap between waves cannot be relied on: the second tile's
                // score product is issued in between the exp2/pack work of the first, and the first
                // tile's value product in between that of the second.  K1 and U^T operands are
                // read once for both tiles; the K1 operands of a block are fetched during the
                // previous block of the same stage.
                // Interior stages [in_lo, in_hi): all 64 keys valid for every (q, k) of both tiles.
                int in_lo = st_lo, in_hi = min(nst, (min(jmax[0], jmax[1]) + 1) / JS);
                if constexpr (WIN) {
                    if (banded) {
                        const int k0 = kt * 32;
                        bool rows_in = true;
                        int lo_key = 0, hi_key = jend;
#pragma unroll
                        for (int t = 0; t < NT; ++t) {
                            rows_in = rows_in && (k0 + 31 <= jmax[t]) && (qrow[t] <= k0 + p.wb);
                            lo_key = max(lo_key, max(qrow[t] - p.wa, k0 + 31 - p.lab));
                            hi_key = min(hi_key, min(jmax[t], k0 + p.rab));
                        }
                        in_lo = min(st_hi + 1, max(st_lo, (lo_key + JS - 1) / JS));
                        in_hi = rows_in ? min(st_hi + 1, max(in_lo, (hi_key + 1) / JS)) : in_lo;
                    }
                }
                // MASKED (the stages that straddle the causal bound or an edge of the band): a key that is
                // not valid for its (q, k) starts its score at -3e4 (C operand of the first k-step), so its P
                // is exactly 0.  Element i of a lane is key jb + key_of(0, i) + 8 g.
                auto fused = [&](auto masked_tag, const E* utp, const E* k1_next, v8 (&kn)[KS], int jb) {
                constexpr bool MASKED = decltype(masked_tag)::value;
                v8 ka[KS], ua[DT][2];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) ka[ks] = kn[ks];
                f32x16 s0, s1;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if constexpr (WIN) {
                        const int j = jb + key_of(0, i) + 8 * g;
                        s0[i] = (MASKED && (j < wlo[0] || j > whi[0])) ? -3.0e4f : 0.f;
                        s1[i] = (MASKED && (j < wlo[1] || j > whi[1])) ? -3.0e4f : 0.f;
                    } else {
                        s0[i] = (MASKED && key_of(0, i) > jmax[0] - jb - 8 * g) ? -3.0e4f : 0.f;
                        s1[i] = (MASKED && key_of(0, i) > jmax[1] - jb - 8 * g) ? -3.0e4f : 0.f;
                    }
                }
                v8 pa0[2], pa1[2];
                // quarter r of a tile's exp2 / pack / row-sum work: 4 exp2, 2 packs, 2 dot2
                auto quarter = [&](const f32x16& sc, v8 (&pa)[2], float& ls, int r) {
                    const int h = r >> 1, e0 = 4 * (r & 1);
#pragma unroll
                    for (int e = e0; e < e0 + 4; e += 2) {
                        const v2 pr = M::pack(fast_exp2(sc[h * 8 + e]), fast_exp2(sc[h * 8 + e + 1]));
                        ls = M::add_pair(pr, ls);
                        pa[h][e] = pr[0];
                        pa[h][e + 1] = pr[1];
                    }
                };
                [[maybe_unused]] v8 lo[KS];
                if constexpr (SPLIT) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) lo[ks] = lo_of(0, ks);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) s0 = M::mma(ka[ks], bq[0][ks], s0);
                if constexpr (SPLIT) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) s0 = M::mma(ka[ks], lo[ks], s0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) lo[ks] = lo_of(1, ks);  // tile 1's, under the products above
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) s1 = M::mma(ka[ks], lo[ks], s1);
                }
                __builtin_amdgcn_sched_barrier(0);
                // U^T operands are first needed two MFMA groups from here
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        ua[dt][h] = *reinterpret_cast<const v8*>(utp + dt * 32 * LDU + h * 16);
                __builtin_amdgcn_sched_barrier(0);
                static_assert(KS == 4 && DT == 2, "the interleave below is written for D = 64");
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    s1 = M::mma(ka[r], bq[1][r], s1);
                    __builtin_amdgcn_sched_barrier(0);
                    quarter(s0, pa0, lsum[0], r);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the K1 operands are dead now: fetch those of the next block (null: none in reach)
                if (k1_next) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) kn[ks] = *reinterpret_cast<const v8*>(k1_next + ks * 16);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[0][r & 1] = M::mma(pa0[r >> 1], ua[r & 1][r >> 1], acc[0][r & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                    quarter(s1, pa1, lsum[1], r);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[1][r & 1] = M::mma(pa1[r >> 1], ua[r & 1][r >> 1], acc[1][r & 1]);
                __builtin_amdgcn_sched_barrier(0);
                };
                auto stage_nt2 = [&](auto masked_tag) {
                    constexpr bool MASKED = decltype(masked_tag)::value;
                    const int sb = gstage & 1;
                    issue_stage(st < st_hi ? st + 1 : st_next);
                    if (st == st_lo && kt + 1 < nkt) issue_ktile(kt + 1);
                    const E* k1p = sK1 + (sb * JS + krow_off) * LDK + g * 8;
                    const E* utp = sUT + (sb * D + n) * LDU + g * 8;
                    v8 kn[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) kn[ks] = *reinterpret_cast<const v8*>(k1p + ks * 16);
                    static_assert(JS == 64 || NT != 2, "two blocks per stage");
                    fused(masked_tag, utp, k1p + 32 * LDK, kn, st * JS);
                    if (!MASKED || st * JS + 32 <= jend) fused(masked_tag, utp + 32, nullptr, kn, st * JS + 32);
                    commit_stage(sb ^ 1);
                    __syncthreads();
                };
                for (; st < in_lo; ++st, ++gstage) stage_nt2(std::true_type{});   // leading edge of the band
                for (; st < in_hi; ++st, ++gstage) stage_nt2(std::false_type{});
                for (; st <= st_hi; ++st, ++gstage) stage_nt2(std::true_type{});  // the diagonal / trailing edge
            }
            if constexpr (NT == 1 && !CAREFUL) {
                // The same for one tile per wave (D = 128: two tiles do not fit the register file).
                // The two 32-key steps of a stage play the part of the two tiles: the score product
                // of the second step is issued between the exp2 / pack work of the first, the value
                // product of the first between that of the second.  No branch on validity inside
                // the loop; every operand is read ahead of its use.
                static_assert(JS == 64, "two steps per stage");
                int nfull = min(nst, (jmax[0] + 1) / JS);
                if constexpr (WIN) {
                    if (banded) {
                        // stages whose 64 keys are inside the band of every (q, k) of this tile; the stages
                        // before them go through the general loop first
                        const int q = qrow[0], k0 = kt * 32;
                        const bool rows_in = (k0 + 31 <= jmax[0]) && (q <= k0 + p.wb);
                        const int in_lo = (max(0, max(q - p.wa, k0 + 31 - p.lab)) + JS - 1) / JS;
                        nfull = rows_in ? min(st_hi + 1, (min(jmax[0], k0 + p.rab) + 1) / JS) : 0;
                        general_until(min(st_hi + 1, max(st_lo, min(in_lo, nfull))));
                    }
                }
                // MASKED (MDIAG: the stages that straddle the causal bound of this wave's query, or lie past it
                // while other waves still need them): a key past the bound starts its score at -3e4, so its P
                // is exactly 0.  Element i of a lane is key jb + key_of(0, i) + 8 g.
                auto stage_nt1 = [&](auto masked_tag) {
                    constexpr bool MASKED = decltype(masked_tag)::value;
                    const int sb = gstage & 1;
                    issue_stage(st < st_hi ? st + 1 : st_next);
                    if (st == st_lo && kt + 1 < nkt) issue_ktile(kt + 1);
                    const E* k1p = sK1 + (sb * JS + krow_off) * LDK + g * 8;
                    const E* utp = sUT + (sb * D + n) * LDU + g * 8;
                    v8 ka[KS], ua[DT][2], pa[2][2];
                    f32x16 sc[2];
                    [[maybe_unused]] const int room = jmax[0] - st * JS - 8 * g;  // keys of this stage inside the bound
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        sc[0][i] = (MASKED && key_of(0, i) > room) ? -3.0e4f : 0.f;
                        sc[1][i] = (MASKED && key_of(0, i) + 32 > room) ? -3.0e4f : 0.f;
                    }
                    auto load_k = [&](int half) {
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks)
                            ka[ks] = *reinterpret_cast<const v8*>(k1p + half * 32 * LDK + ks * 16);
                    };
                    // U^T operands of key half `half`, k-step h: fetched as soon as the registers they take over
                    // (K1 operands, or the other half's U^T operands) have been issued to their last MFMA
                    auto load_u = [&](int half, int h) {
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
                            ua[dt][h] = *reinterpret_cast<const v8*>(utp + half * 32 + dt * 32 * LDU + h * 16);
                    };
                    auto pair = [&](int half, int r) {  // register pair r (0..7): 2 exp2, 1 pack, 1 row-sum step
                        const int h = r >> 2, e = 2 * (r & 3);
                        const v2 pr = M::pack(fast_exp2(sc[half][h * 8 + e]), fast_exp2(sc[half][h * 8 + e + 1]));
                        lsum[0] = M::add_pair(pr, lsum[0]);
                        pa[half][h][e] = pr[0];
                        pa[half][h][e + 1] = pr[1];
                    };
                    auto value_mma = [&](int half, int r) {  // r = 0 .. 2 DT - 1; dependent ones are DT apart
                        const int h = r / DT, dt = r % DT;
                        acc[0][dt] = M::mma(pa[half][h], ua[dt][h], acc[0][dt]);
                    };
                    load_k(0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        sc[0] = M::mma(ka[ks], bq[0][ks], sc[0]);
                        if constexpr (SPLIT) sc[0] = M::mma(ka[ks], lo_of(0, ks), sc[0]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    load_k(1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        sc[1] = M::mma(ka[ks], bq[0][ks], sc[1]);
                        if constexpr (SPLIT) sc[1] = M::mma(ka[ks], lo_of(0, ks), sc[1]);
                        __builtin_amdgcn_sched_barrier(0);
                        if (ks == KS / 2 - 1) load_u(0, 0);
#pragma unroll
                        for (int r = ks * 8 / KS; r < (ks + 1) * 8 / KS; ++r) pair(0, r);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    load_u(0, 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 2 * DT; ++r) {
                        value_mma(0, r);
                        __builtin_amdgcn_sched_barrier(0);
                        if (r == DT - 1) load_u(1, 0);
#pragma unroll
                        for (int q2 = r * 8 / (2 * DT); q2 < (r + 1) * 8 / (2 * DT); ++q2) pair(1, q2);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    load_u(1, 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 2 * DT; ++r) value_mma(1, r);
                    __builtin_amdgcn_sched_barrier(0);
                    commit_stage(sb ^ 1);
                    __syncthreads();
                };
                for (; st < nfull; ++st, ++gstage) stage_nt1(std::false_type{});
                if constexpr (MDIAG && !WIN) {
                    for (; st <= st_hi; ++st, ++gstage) stage_nt1(std::true_type{});
                }
            }
            general_until(st_hi + 1);
        };

        sweep(std::false_type{});
        bool redone = false;
        {
            // did any valid virtual row of this workgroup leave the safe range?
            bool bad = false;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                // every P is at most its row sum, so a row sum inside this range keeps the value accumulators
                // (P times SiLU(V1), a handful of terms) finite as well
                const float lk = lsum[t] + __shfl_xor(lsum[t], 32, 64);
                bool kval = (kt * 32 + n) <= jmax[t];
                if constexpr (WIN) kval = whi[t] >= 0;
                bad |= kval && !(lk > fast_row_sum_floor<E>() && lk < 1e25f);
            }
            // One barrier per k-tile: this k-tile's flag is read after it; the other flag was read by every
            // wave before it arrived here, is cleared now, and is next written after the barriers of the
            // following k-tile's sweep.
            if (__any(bad) && lane == 0) sFlag[kb] = 1;
            // The next k-tile's K2 / V2 rows go to LDS here too (their buffer was last read in the previous
            // k-tile, and every wave has crossed a stage barrier of this one since), so the same barrier
            // publishes them and the k-tile needs none at its end.
            if (kt + 1 < nkt) commit_ktile(kb ^ 1);
            __syncthreads();
            const bool redo = sFlag[kb] != 0;
            if (tid == 0) sFlag[kb ^ 1] = 0;
            if (redo) {
                if constexpr (WIN) {
                    if (st_next != st_lo) {  // the stage fetched ahead belongs to the next k-tile: fetch this one's
                        issue_stage(st_lo);
                        commit_stage(gstage & 1);
                        __syncthreads();
                    }
                }
                sweep(std::true_type{});
                redone = true;
            }
        }

        // ---- merge the 32 virtual rows (q, k) of each tile into the running O[q] -------------
        // The common case first: this k-tile and every one before it kept the reference at 0 (FAST sweeps), so
        // every weight is 1 and nothing is rescaled: O += sum_k V2[k] (.) Tv[(q, k)], L += sum_k l_k over the
        // valid rows.  Only the diagonal k-tile holds rows past the causal bound; it clears them first.
        if constexpr (!WIN) {
            plain = plain && !redone;
            if (plain) {
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const float lk = lsum[t] + __shfl_xor(lsum[t], 32, 64);
                    const bool kval = (kt * 32 + n) <= jmax[t];
                    float wl = kval ? lk : 0.f;
#pragma unroll
                    for (int off = 16; off > 0; off >>= 1) wl += __shfl_xor(wl, off, 64);
                    Lrun[t] += wl;
                    Mrun[t] = 0.f;
                    if (!__all(kval)) {
                        float wr[16];
                        rows_of(kval ? 1.f : 0.f, wr);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                            for (int i = 0; i < 16; ++i) acc[t][dt][i] = wr[i] == 0.f ? 0.f : acc[t][dt][i];
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        float part = 0.f;
#pragma unroll
                        for (int i = 0; i < 16; ++i)
                            part += (float)sV2[(kb * 32 + c_row(g, i)) * LDK + dt * 32 + n] * acc[t][dt][i];
                        Orun[t][dt] += part;
                    }
                }
                continue;
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float lk = lsum[t] + __shfl_xor(lsum[t], 32, 64);
            bool kval = (kt * 32 + n) <= jmax[t];
            if constexpr (WIN) kval = whi[t] >= 0;
            float mt = kval ? mref[t] : -INFINITY;
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) mt = fmaxf(mt, __shfl_xor(mt, off, 64));
            const float mnew = fmaxf(Mrun[t], mt);
            // WIN: the first k-tiles of the band can hold no valid row for this query yet
            const float f = (WIN && mnew == -INFINITY) ? 1.f : fast_exp2(Mrun[t] - mnew);
            const float w = kval ? fast_exp2(mref[t] - mnew) : 0.f;
            float wl = kval ? w * lk : 0.f;  // a row past the causal bound was swept unmasked: its sum may be inf
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) wl += __shfl_xor(wl, off, 64);
            Lrun[t] = Lrun[t] * f + wl;
            Mrun[t] = mnew;
            float wr[16];
            rows_of(w, wr);
            // wr = 0 for rows outside the mask.  The FAST sweep ran them unmasked and unchecked, so their
            // accumulators may hold inf or NaN (fp16 tensors: exp2 of a score above 16 is inf) and 0 * inf must
            // not reach the sum: k-tiles that hold such rows (the diagonal one, the edges of a band) clear them.
            if (!__all(kval)) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[t][dt][i] = wr[i] == 0.f ? 0.f : acc[t][dt][i];
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                float part = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float v = (float)sV2[(kb * 32 + c_row(g, i)) * LDK + dt * 32 + n];
                    part += wr[i] * v * acc[t][dt][i];
                }
                Orun[t][dt] = Orun[t][dt] * f + part;
            }
        }

    }

    // ---- epilogue ---------------------------------------------------------------------------
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int q = qrow[t];
        if (p.splits > 1) {
            float* dst = p.part + (((size_t)bh * T + q) * p.splits + split) * (D + 2);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const float o = Orun[t][dt] + __shfl_xor(Orun[t][dt], 32, 64);
                if (q < T && g == 0) dst[dt * 32 + n] = o;
            }
            if (q < T && lane == 0) {
                dst[D] = Mrun[t];
                dst[D + 1] = Lrun[t];
            }
            continue;
        }
        const float inv = 1.0f / Lrun[t];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const float o = (Orun[t][dt] + __shfl_xor(Orun[t][dt], 32, 64)) * inv;
            if (q < T && g == 0) {
                const E rounded = (E)o;
                p.o[base + (size_t)q * D + dt * 32 + n] = rounded;
                if constexpr (SPLIT) p.o_res[base + (size_t)q * D + dt * 32 + n] = (E)(o - (float)rounded);
            }
        }
        if (q < T && lane == 0) p.lse[(size_t)bh * T + q] = (Mrun[t] + fast_log2(Lrun[t])) * kLn2;
    }
}

// Joins the parts a split forward left behind: one thread per (row, d).
template <typename E>
__global__ __launch_bounds__(256) void fwd_merge_kernel(const float* __restrict__ part, E* __restrict__ o,
                                                        E* __restrict__ o_res, float* __restrict__ lse, int rows,
                                                        int D, int splits) {
    // 64-bit element index: rows * D can pass 2^31 (the forced-split override applies at any size)
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t row = idx / D;
    const int d = (int)(idx % D);
    if (row >= (size_t)rows) return;
    const float* src = part + row * splits * (D + 2);
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, src[s * (D + 2) + D]);
    float l = 0.f, acc = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float ms = src[s * (D + 2) + D];
        if (ms == -INFINITY) continue;  // an empty part: its other fields were never written
        const float w = fast_exp2(ms - m);
        l += w * src[s * (D + 2) + D + 1];
        acc += w * src[s * (D + 2) + d];
    }
    const float out = acc / l;
    const E rounded = (E)out;
    o[row * D + d] = rounded;
    if (o_res) o_res[row * D + d] = (E)(out - (float)rounded);  // split operands: see tdp_fwd_mfma_kernel
    if (d == 0) lse[row] = (m + fast_log2(l)) * kLn2;
}

// U^T[bh][d][j] = SiLU(V1[bh][j][d]) for j < T, 0 for T <= j < Tp
template <typename E>
__global__ __launch_bounds__(256) void silu_transpose_kernel(const E* __restrict__ v1, E* __restrict__ ut, int T,
                                                             int Tp, int D, int H, long long sb, long long sh,
                                                             unsigned st) {
    const int bh = blockIdx.y, j0 = blockIdx.x * 64;
    __shared__ E tile[64 * (128 + 2)];
    transpose_load<E, true>(v1 + (size_t)(bh / H) * sb + (size_t)(bh % H) * sh, nullptr, tile, j0, T, D, st);
    __syncthreads();
    transpose_store<E>(ut + (size_t)bh * D * Tp, tile, j0, Tp, D);
}

template <int D, int NT, int WAVES, int JS, bool SPLIT = false>
constexpr size_t fwd_smem_bytes() {
    return sizeof(uint16_t) * (2 * JS * (D + 8) + 2 * D * (JS + 8) + 4 * 32 * (D + 8)) +
           sizeof(float) * (WAVES * NT * (D + 4) + WAVES * 32) + 16 +
           (SPLIT ? sizeof(uint16_t) * WAVES * NT * (D / 16) * 512 : 0);
}

}  // namespace tritt
#include "tdp_fwd_band.hpp"
namespace tritt {

constexpr int kTpad = 128;  // U^T rows are padded to a multiple of the largest stage

// Small grids split the k-tiles of every query tile over several workgroups: a causal grid ends in its heaviest
// query tiles, three times the average, and one workgroup fills a CU.  Measured optimum: enough parts for about
// 768 workgroups, no more than 4 (every part pays the prologue and a tail), and parts of at least 2 k-tiles
// (4 under a windowed mask, whose k-tiles see only a few steps of j each).
constexpr int kFwdSplitTarget = 768, kAutoFwdSplits = 4, kMaxFwdSplits = 8;

// queries per workgroup of the instantiation mfma_tdp_fwd() picks: D = 64 runs two queries per wave, the others one
static int fwd_tile_queries(int D, int /*windowed*/) { return D == 64 ? 16 : 8; }

static size_t ut_bytes(int BH, int T, int D) {
    const size_t Tp = (size_t)(T + kTpad - 1) / kTpad * kTpad;
    return ((size_t)BH * D * Tp * 2 + 255) / 256 * 256;
}

// TRITT_FWD_SPLITS overrides the count (tests, tuning sweeps); read once per process (knobs())
// The band-resident kernel takes windowed causal masks whose band fits in LDS (with room to spare for the
// compiler's own use).  TRITT_FWD_BAND=0 switches it off (A/B runs).
constexpr size_t kBandSmemLimit = 156 * 1024;
static bool use_band_kernel(const MfmaFwdArgs& a) {
    if (!(a.windowed && a.causal)) return false;
    if (a.split) return false;  // split operands: the streaming kernels only
    if (knobs().fwd_band < 0) return false;
    const int nr = band_rows(a.k1_window, a.k2_window);
    const size_t smem = a.D == 32 ? band_smem_bytes<32>(nr) : a.D == 64 ? band_smem_bytes<64>(nr) : band_smem_bytes<128>(nr);
    return smem <= kBandSmemLimit;
}

// The layout the kernels are handed: the caller's strides, or those of a dense [BH][T][D] tensor (in_st == 0)
struct InLayout {
    long long sb, sh;
    unsigned st;
    int H;
};
static InLayout input_layout(const MfmaFwdArgs& a, bool of_v1) {
    const long long st = of_v1 ? a.v1_st : a.in_st;
    if (st == 0) return {(long long)a.T * a.D, 0, (unsigned)a.D, 1};  // dense: batch and head are one index
    return of_v1 ? InLayout{a.v1_sb, a.v1_sh, (unsigned)a.v1_st, a.H} : InLayout{a.in_sb, a.in_sh, (unsigned)a.in_st, a.H};
}

template <typename E, int D>
static hipError_t launch_band(const MfmaFwdArgs& a, hipStream_t st) {
    const int Tp = (a.T + kTpad - 1) / kTpad * kTpad;
    const InLayout lin = input_layout(a, false), lv1 = input_layout(a, true);
    hipLaunchKernelGGL(silu_transpose_kernel<E>, dim3(Tp / 64, a.BH), dim3(256), 0, st, (const E*)a.v1, (E*)a.ut,
                       a.T, Tp, D, lv1.H, lv1.sb, lv1.sh, lv1.st);
    FwdParams<E> p;
    p.q = (const E*)a.q; p.k1 = (const E*)a.k1; p.k2 = (const E*)a.k2; p.v2 = (const E*)a.v2;
    p.ut = (const E*)a.ut; p.o = (E*)a.o; p.lse = a.lse; p.o_res = nullptr;
    p.in_sb = lin.sb; p.in_sh = lin.sh; p.in_st = lin.st; p.H = lin.H;
    p.T = a.T; p.Tp = Tp; p.BH = a.BH; p.nqt = (a.T + kBandQ - 1) / kBandQ;
    p.scale_log2 = a.alpha * kLog2e;
    p.causal = 1;
    p.wa = a.k1_window; p.wb = a.k2_window; p.lab = a.kk_left; p.rab = a.kk_right;
    p.splits = 1;
    p.part = nullptr;
    const int nr = band_rows(p.wa, p.wb);
    const size_t smem = band_smem_bytes<D>(nr);
    auto kern = a.many_views ? tdp_fwd_band_kernel<E, D, true> : tdp_fwd_band_kernel<E, D, false>;
    p.at_k1 = a.at_k1; p.at_k2 = a.at_k2; p.at_v2 = a.at_v2;
    hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, p.nqt)), dim3(512), smem, st, p, nr);
    return hipGetLastError();
}

static int fwd_splits(const MfmaFwdArgs& a, int bq) {
    if (use_band_kernel(a)) return 1;
    if (knobs().fwd_splits > 0) return min(knobs().fwd_splits, kMaxFwdSplits);
    const int wgs = a.BH * ((a.T + bq - 1) / bq);
    const bool banded = a.windowed && a.causal;
    // keys k the heaviest query tile walks
    const int span = banded ? min(a.T, max(a.k2_window, a.k1_window + a.kk_right) + bq) : a.T;
    const int by_size = (kFwdSplitTarget + wgs - 1) / wgs, by_tiles = (span + 31) / 32 / (banded ? 4 : 2);
    return max(1, min(kAutoFwdSplits, min(by_size, by_tiles)));
}

template <typename E, int D, int NT, int WAVES, int MINW, int JS, bool WIN = false, bool MDIAG = false, bool SPLIT = false>
static hipError_t launch(const MfmaFwdArgs& a, hipStream_t st) {
    const int Tp = (a.T + kTpad - 1) / kTpad * kTpad;
    const InLayout lin = input_layout(a, false), lv1 = input_layout(a, true);
    hipLaunchKernelGGL(silu_transpose_kernel<E>, dim3(Tp / 64, a.BH), dim3(256), 0, st, (const E*)a.v1, (E*)a.ut,
                       a.T, Tp, D, lv1.H, lv1.sb, lv1.sh, lv1.st);
    constexpr int BQ = WAVES * NT;
    if (BQ != fwd_tile_queries(D, a.windowed)) return hipErrorInvalidValue;  // the workspace was sized for another shape
    FwdParams<E> p;
    p.q = (const E*)a.q; p.k1 = (const E*)a.k1; p.k2 = (const E*)a.k2; p.v2 = (const E*)a.v2;
    p.ut = (const E*)a.ut; p.o = (E*)a.o; p.lse = a.lse;
    p.in_sb = lin.sb; p.in_sh = lin.sh; p.in_st = lin.st; p.H = lin.H;
    p.o_res = SPLIT ? (E*)a.o + (size_t)a.BH * a.T * D : nullptr;
    p.T = a.T; p.Tp = Tp; p.BH = a.BH; p.nqt = (a.T + BQ - 1) / BQ;
    p.scale_log2 = a.alpha * kLog2e;
    p.causal = a.causal;
    p.wa = a.k1_window; p.wb = a.k2_window; p.lab = a.kk_left; p.rab = a.kk_right;
    p.splits = fwd_splits(a, BQ);
    p.part = reinterpret_cast<float*>(static_cast<char*>(a.ut) + ut_bytes(a.BH, a.T, D));
    constexpr size_t smem = fwd_smem_bytes<D, NT, WAVES, JS, SPLIT>();
    auto kern = a.many_views ? tdp_fwd_mfma_kernel<E, D, NT, WAVES, MINW, JS, WIN, MDIAG, SPLIT, true>
                             : tdp_fwd_mfma_kernel<E, D, NT, WAVES, MINW, JS, WIN, MDIAG, SPLIT, false>;
    p.at_k1 = a.at_k1; p.at_k2 = a.at_k2; p.at_v2 = a.at_v2;
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, p.nqt) * p.splits), dim3(64 * WAVES), smem, st, p);
    if (p.splits > 1) {
        const int rows = a.BH * a.T;
        hipLaunchKernelGGL(fwd_merge_kernel<E>, dim3((unsigned)(((size_t)rows * D + 255) / 256)), dim3(256), 0, st,
                           p.part, (E*)a.o, p.o_res, a.lse, rows, D, p.splits);
    }
    return hipGetLastError();
}

// U^T, then the parts of a split forward
size_t mfma_tdp_fwd_workspace(const MfmaFwdArgs& a) {
    const int splits = fwd_splits(a, fwd_tile_queries(a.D, a.windowed));
    return ut_bytes(a.BH, a.T, a.D) + (splits > 1 ? (size_t)a.BH * a.T * splits * (a.D + 2) * sizeof(float) : 0);
}

bool mfma_tdp_fwd_supported(int D, int dtype_is_16bit) { return dtype_is_16bit && (D == 32 || D == 64 || D == 128); }
bool mfma_tdp_split_supported(int D, int dtype_is_16bit) { return dtype_is_16bit && (D == 32 || D == 64); }

template <typename E>
static hipError_t launch_split(const MfmaFwdArgs& a, hipStream_t st) {
    if (a.windowed) {
        if (a.D == 32) return launch<E, 32, 1, 8, 2, 64, true, false, true>(a, st);
        if (a.D == 64) return launch<E, 64, 2, 8, 2, 64, true, false, true>(a, st);
    } else {
        if (a.D == 32) return launch<E, 32, 1, 8, 2, 64, false, false, true>(a, st);
        if (a.D == 64) return launch<E, 64, 2, 8, 2, 64, false, false, true>(a, st);
    }
    return hipErrorInvalidValue;
}

hipError_t mfma_tdp_fwd(const MfmaFwdArgs& a, hipStream_t st) {
    if (a.split) return a.is_bf16 ? launch_split<__bf16>(a, st) : launch_split<_Float16>(a, st);
    if (use_band_kernel(a)) {
        if (a.is_bf16) {
            if (a.D == 32) return launch_band<__bf16, 32>(a, st);
            if (a.D == 64) return launch_band<__bf16, 64>(a, st);
            if (a.D == 128) return launch_band<__bf16, 128>(a, st);
        } else {
            if (a.D == 32) return launch_band<_Float16, 32>(a, st);
            if (a.D == 64) return launch_band<_Float16, 64>(a, st);
            if (a.D == 128) return launch_band<_Float16, 128>(a, st);
        }
        return hipErrorInvalidValue;
    }
    if (a.windowed) {
        // one tile per wave, eight waves: the stages inside the band run the two-step interleaved loop,
        // the stages on its edges the general one
        if (a.is_bf16) {
            if (a.D == 32) return launch<__bf16, 32, 1, 8, 2, 64, true>(a, st);
            if (a.D == 64) return launch<__bf16, 64, 2, 8, 2, 64, true>(a, st);
            if (a.D == 128) return launch<__bf16, 128, 1, 8, 2, 64, true>(a, st);
        } else {
            if (a.D == 32) return launch<_Float16, 32, 1, 8, 2, 64, true>(a, st);
            if (a.D == 64) return launch<_Float16, 64, 2, 8, 2, 64, true>(a, st);
            if (a.D == 128) return launch<_Float16, 128, 1, 8, 2, 64, true>(a, st);
        }
        return hipErrorInvalidValue;
    }
    if (a.is_bf16) {
        if (a.D == 32) return launch<__bf16, 32, 1, 8, 2, 64>(a, st);
        if (a.D == 64) return launch<__bf16, 64, 2, 8, 2, 64>(a, st);
        if (a.D == 128) return launch<__bf16, 128, 1, 8, 2, 64>(a, st);
    } else {
        if (a.D == 32) return launch<_Float16, 32, 1, 8, 2, 64>(a, st);
        if (a.D == 64) return launch<_Float16, 64, 2, 8, 2, 64>(a, st);
        if (a.D == 128) return launch<_Float16, 128, 1, 8, 2, 64>(a, st);
    }
    return hipErrorInvalidValue;
}

}  // namespace tritt
