// The device side of the fp32 matrix-core triple-dot kernels (tdp_f32_mfma.hip holds the description and the launchers),
// as a header: the 16-bit backward appends the workgroups of its fp32 query tile 0 to the grid of its own first launch
// (tdp_bwd_mfma.hip), so both translation units instantiate these bodies.
#pragma once
#include <algorithm>

#include "common.hpp"
#include "kernels.hpp"
#include "mfma.hpp"

namespace tritt {
namespace {

constexpr int kF32Waves = 8;
constexpr float kNegBig = -1.0e30f;  // finite stand-in for "no maximum yet"

__device__ __forceinline__ f32x16 mma_f32(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <typename E>
struct F32Params {
    const E *q, *ka, *kb, *va, *vb;  // streamed = (ka, va), rows = (kb, vb)
    // where these five and d_o lie: H heads per batch entry and each tensor's strides (dense tensors: H = 1 and
    // sb = T D, st = D); the outputs are dense
    int H;
    TensorAt at_q, at_ka, at_kb, at_va, at_vb, at_do;
    E* o;
    float* lse;
    // STATS mode (the 16-bit backward's fp32 tiles): O is not written; lse receives the fp32 log-sum-exp of the
    // covered rows and delta their rowsum(dO * O) with O in fp32
    const E* d_o;
    float* delta;
    // STATS over query tile 0 with the rounds dealt out to `split_rounds` workgroups (blockIdx.y): each writes its
    // partial (maximum, sum, sum_d dO * unnormalised O) to delta[((bh * 32 + q) * split_rounds + round) * 3 ..] and
    // the first one clears `zero_words` 4-byte words at zero_ptr + bh * zero_words
    int split_rounds;
    unsigned* zero_ptr;
    int zero_words;
    int T, BH, nqt;  // nqt: query tiles this launch covers (tiles 0 .. nqt - 1)
    float scale_log2;
    TdpMask mask;  // in terms of the streamed index a and the row index b
};

// Ranges of streamed rows / owner rows a tile of queries [q0, q1] can touch.
struct Range {
    int lo, hi;
};
__device__ __forceinline__ Range row_range(const TdpMask& m, int q0, int q1, int T) {
    if (!m.causal) return {0, T - 1};
    return {max(0, q0 - m.wb), q1};
}
__device__ __forceinline__ Range streamed_range(const TdpMask& m, int q0, int q1, int b, int T) {
    if (!m.causal) return {0, T - 1};
    // a <= q, q - a <= wa, b - a <= lab, a - b <= rab
    return {max(0, max(q0 - m.wa, b - m.lab)), min(q1, b + m.rab)};
}

// Staging of 32 x D tiles of E through registers (16-byte pieces), converted to fp32 on the way into LDS.
template <typename E, int D>
struct StageE {
    static constexpr int VE = 16 / (int)sizeof(E);           // elements per piece
    static constexpr int kPieces = 32 * D / VE;               // per tensor
    static constexpr int kPer = (kPieces + 255) / 256;        // per thread
    uint4 x[kPer];
};
template <typename E, int D>
__device__ __forceinline__ void stage_fetch_e(StageE<E, D>& r, const E* __restrict__ ka, const E* __restrict__ va, int a0,
                                              int T, unsigned pitch_ka, unsigned pitch_va) {
    using S = StageE<E, D>;
    constexpr int kVec = D / S::VE;
    const int t = threadIdx.x & 255;
    const E* src = threadIdx.x < 256 ? ka : va;
    const unsigned pitch = threadIdx.x < 256 ? pitch_ka : pitch_va;
#pragma unroll
    for (int i = 0; i < S::kPer; ++i) {
        const int idx = t + i * 256;
        if (idx < S::kPieces) {
            const int row = idx / kVec, c = idx % kVec;
            r.x[i] = *reinterpret_cast<const uint4*>(src + (size_t)min(a0 + row, T - 1) * pitch + c * S::VE);
        }
    }
}
template <typename E, int D>
__device__ __forceinline__ void stage_store_e(const StageE<E, D>& r, float* sk, float* sv) {
    using S = StageE<E, D>;
    constexpr int kVec = D / S::VE, LD = D + 1;
    const int t = threadIdx.x & 255;
    float* dst = threadIdx.x < 256 ? sk : sv;
#pragma unroll
    for (int i = 0; i < S::kPer; ++i) {
        const int idx = t + i * 256;
        if (idx < S::kPieces) {
            const int row = idx / kVec, c = idx % kVec;
            float* p = dst + row * LD + c * S::VE;
            const E* e = reinterpret_cast<const E*>(&r.x[i]);
#pragma unroll
            for (int k = 0; k < S::VE; ++k) p[k] = (float)e[k];
        }
    }
}

// ------------------------------------------------------------------------------------------ forward
template <typename E, int D, bool STATS>
__global__ __launch_bounds__(512) void tdp_f32_fwd_kernel(F32Params<E> p) {
    constexpr int DT = D / 32, KS = D / 2, LD = D + 1, NW = kF32Waves;
    constexpr bool FLY = D > 64;  // form the B operand of the score product as it is used
    extern __shared__ __align__(16) float smem_f[];
    float* sK = smem_f;                 // [2][32][LD] streamed key rows
    float* sV = sK + 2 * 32 * LD;       // [2][32][LD] streamed value rows
    float* sQ = sV + 2 * 32 * LD;       // [32][LD]    the tile's queries * scale
    float* sKb = sQ + 32 * LD;          // [NW][D]     row operands of the round
    float* sVb = sKb + NW * D;          // [NW][D]
    float* sM = sVb + NW * D;           // [NW][32]    end of kernel: per-wave maxima and sums
    float* sL = sM + NW * 32;           // [NW][32]
    float* sO = sK;                     // [D][33]     end of kernel: merged output (aliases the stages)

    int bh, order;
    if (!xcd_tile(p.BH, p.nqt, blockIdx.x >> 3, blockIdx.x & 7, bh, order)) return;
    const int qt = p.nqt - 1 - order;  // heaviest query tiles first

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D;
    const int b_ = bh / p.H, h_ = bh % p.H;
    auto slice = [&](const E* t, const TensorAt& at) { return t + (size_t)b_ * at.sb + (size_t)h_ * at.sh; };
    const E* __restrict__ KA = slice(p.ka, p.at_ka);
    const E* __restrict__ VA = slice(p.va, p.at_va);
    const E* __restrict__ KB = slice(p.kb, p.at_kb);
    const E* __restrict__ VB = slice(p.vb, p.at_vb);
    const E* __restrict__ Qs = slice(p.q, p.at_q);
    const TdpMask mask = p.mask;

    const int q0 = qt * 32, q1 = min(T - 1, q0 + 31);
    const int q = q0 + n;  // this lane's query (column of every tile)
    for (int idx = tid; idx < 32 * D; idx += 512) {
        const int r = idx / D, d = idx % D;
        sQ[r * LD + d] = (float)Qs[(size_t)min(q0 + r, T - 1) * p.at_q.st + d] * p.scale_log2;
    }

    const Range rows = row_range(mask, q0, q1, T);
    int m_lo = rows.lo / NW, m_hi = rows.hi / NW;  // rounds of NW rows
    if (STATS && p.split_rounds) {
        m_lo = max(m_lo, (int)blockIdx.y);  // this workgroup's round only (none at all if it is out of range)
        m_hi = min(m_hi, (int)blockIdx.y);
        if (blockIdx.y == 0)
            for (int idx = tid; idx < p.zero_words; idx += 512) p.zero_ptr[(size_t)bh * p.zero_words + idx] = 0u;
    }

    f32x16 accO[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) accO[dt][i] = 0.f;
    float m_run = kNegBig, l_run = 0.f;  // per query, over every (a, b) this wave has seen (l: this lane's half)

    StageE<E, D> regs;
    for (int m = m_lo; m <= m_hi; ++m) {
        const int b = m * NW + wave;
        // the streamed stages this round needs: the union over its rows
        const Range ra = streamed_range(mask, q0, q1, min(m * NW, T - 1), T);
        const Range rb = streamed_range(mask, q0, q1, min(m * NW + NW - 1, T - 1), T);
        const int st_lo = min(ra.lo, rb.lo) / 32, st_hi = max(ra.hi, rb.hi) / 32;
        const bool row_ok = b <= rows.hi && b >= rows.lo;
        const Range mine = streamed_range(mask, q0, q1, min(b, T - 1), T);

        __syncthreads();  // previous round: everyone is done with sKb / sVb and the stage buffers
        for (int idx = tid; idx < NW * D; idx += 512) {
            const int r = idx / D, d = idx % D;
            const size_t row = (size_t)min(m * NW + r, T - 1);
            sKb[idx] = (float)KB[row * p.at_kb.st + d];
            sVb[idx] = (float)VB[row * p.at_vb.st + d];
        }
        if (st_lo <= st_hi) {
            stage_fetch_e<E, D>(regs, KA, VA, st_lo * 32, T, p.at_ka.st, p.at_va.st);
            stage_store_e<E, D>(regs, sK, sV);
        }
        __syncthreads();

        // B operand of the score product: lane (q, g), step s holds scale * Q[q, g*D/2 + s] * KB[b, g*D/2 + s]
        float bq[FLY ? 1 : KS];
        if constexpr (!FLY) {
#pragma unroll
            for (int s = 0; s < KS; ++s) bq[s] = sQ[n * LD + g * KS + s] * sKb[wave * D + g * KS + s];
        }

        f32x16 accT[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) accT[dt][i] = 0.f;

        for (int st = st_lo; st <= st_hi; ++st) {
            const int buf = (st - st_lo) & 1;
            const float* cK = sK + buf * 32 * LD;
            const float* cV = sV + buf * 32 * LD;
            const bool more = st < st_hi;
            if (more) stage_fetch_e<E, D>(regs, KA, VA, (st + 1) * 32, T, p.at_ka.st, p.at_va.st);
            const int a0 = st * 32;
            if (row_ok && a0 + 31 >= mine.lo && a0 <= mine.hi) {
                f32x16 s;
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int col = g * KS + ks;
                    const float oq = FLY ? sQ[n * LD + col] * sKb[wave * D + col] : bq[FLY ? 0 : ks];
                    s = mma_f32(cK[n * LD + col], oq, s);
                }
                // mask, tile maximum of this lane's 16 rows
                float tmax = kNegBig;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int a = a0 + c_row(g, i);
                    const bool ok = a < T && tdp_valid(mask, q, a, b);
                    s[i] = ok ? s[i] : -INFINITY;
                    tmax = fmaxf(tmax, s[i]);
                }
                tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
                const float m_new = fmaxf(m_run, tmax);
                if (__any(m_new > m_run)) {
                    const float sc = fast_exp2(m_run - m_new);
                    l_run *= sc;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            accT[dt][i] *= sc;
                            accO[dt][i] *= sc;
                        }
                    m_run = m_new;
                }
                float psum = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = fast_exp2(s[i] - m_run);
                    psum += s[i];
                }
                l_run += psum;
                // Tv^T[d, q] += VA^T[d, a] P^T[a, q]: step i contracts the two streamed rows c_row(0, i), c_row(1, i)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) accT[dt] = mma_f32(cV[c_row(g, i) * LD + dt * 32 + n], s[i], accT[dt]);
            }
            if (more) {
                stage_store_e<E, D>(regs, sK + (buf ^ 1) * 32 * LD, sV + (buf ^ 1) * 32 * LD);
                __syncthreads();
            }
        }
        // the finished row: O^T[d, q] += Tv^T[d, q] * VB[b, d]   (register i of half g is d = 32 dt + c_row(g, i))
        if (row_ok) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) accO[dt][i] += accT[dt][i] * sVb[wave * D + dt * 32 + c_row(g, i)];
        }
    }

    // ---- merge the eight waves' partial results (each relative to its own maximum), one wave after another
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();
    if (g == 0) {
        sM[wave * 32 + n] = m_run;
        sL[wave * 32 + n] = l_run;
    }
    for (int idx = tid; idx < D * 33; idx += 512) sO[idx] = 0.f;
    __syncthreads();
    float M = kNegBig;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sM[w * 32 + n]);
    const float mine_scale = fast_exp2(m_run - M);
    for (int w = 0; w < NW; ++w) {
        if (wave == w) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) sO[(dt * 32 + c_row(g, i)) * 33 + n] += accO[dt][i] * mine_scale;
        }
        __syncthreads();
    }
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) L += sL[w * 32 + n] * fast_exp2(sM[w * 32 + n] - M);
    if constexpr (STATS) {
        // Delta[q] = sum_d dO[q, d] O[q, d] with O in fp32 (lane n of wave 0 walks its query's row)
        if (wave == 0 && g == 0 && q < T) {
            float dsum = 0.f;
            for (int d = 0; d < D; ++d) dsum += (float)slice(p.d_o, p.at_do)[(size_t)q * p.at_do.st + d] * sO[d * 33 + n];
            if (p.split_rounds) {
                float* part = p.delta + (((size_t)bh * 32 + n) * p.split_rounds + blockIdx.y) * 3;
                part[0] = M; part[1] = L; part[2] = dsum;
            } else {
                p.delta[(size_t)bh * T + q] = dsum / L;
            }
        }
        if (p.split_rounds) return;
    } else {
        for (int idx = tid; idx < 32 * D; idx += 512) {
            const int r = idx / D, d = idx % D;
            if (q0 + r < T) {
                float Lr = 0.f, Mr = kNegBig;
#pragma unroll
                for (int w = 0; w < NW; ++w) Mr = fmaxf(Mr, sM[w * 32 + r]);
#pragma unroll
                for (int w = 0; w < NW; ++w) Lr += sL[w * 32 + r] * fast_exp2(sM[w * 32 + r] - Mr);
                p.o[base + (size_t)(q0 + r) * D + d] = (E)(sO[d * 33 + r] / Lr);
            }
        }
    }
    if (wave == 0 && g == 0 && q < T) p.lse[(size_t)bh * T + q] = (M + fast_log2(L)) * kLn2;
}

// ------------------------------------------------------------------------------------------ backward
// Launched twice, like the 16-bit backward: rows = (K2, V2), streamed = (K1, U) gives dQ, dK2, dV2; with the roles
// exchanged, dK1 and dU.  Per (query tile, row b, 32 streamed rows):
//   S^T, dP^T (D / 2 MFMAs each),  P = exp2(S - LSE2[q]),  dS = P (dP - Delta[q])   (both lane-local)
//   Yq^T[d, q] += KA^T[d, a] dS^T[a, q]      Tv^T[d, q] += VA^T[d, a] P^T[a, q]      (DOUT / 2 MFMAs each)
// and when the row is finished
//   dQ^T[d, q] += Yq^T[d, q] KB[b, d]                                  (registers, all rounds)
//   dKB[b, d]  += alpha sum_q Yq^T[d, q] Q[q, d],   dVB[b, d] += sum_q Tv^T[d, q] dO[q, d]
// The sums over the tile's 32 queries are lane reductions; the sums over query tiles (workgroups) go to shared
// accumulators: 64-bit fixed point with integer atomics (the result does not depend on the order of arrival), or
// fp32 atomics when the caller's accumulators are fp32.
//
// The tensors may be 16-bit (E = bf16 / f16): they are converted as they are staged, everything after that is
// fp32.  That is how the 16-bit backward runs its first query tile: for the first few causal queries the softmax
// is nearly one-hot and dS = P (dP - Delta) cancels two O(10) numbers, which the 16-bit operands of the MFMA
// kernels (dO * V2 rounded to 16 bit) cannot resolve.
// D = 128: a workgroup produces DOUT = 64 of the gradient columns (blockIdx.y picks the half), and the B operands
// of the score products are formed as they are used instead of being held in registers.
// the fp32 tensors' accumulators resolve 2^-36 of the slice's max |dO| and cover sums up to 2^27 times it
constexpr int kF32FixedBias = 36;

template <typename E>
struct F32BwdParams {
    const E *q, *d_o, *ka, *kb, *va, *vb;
    int H;  // layouts of the six inputs, as in F32Params
    TensorAt at_q, at_ka, at_kb, at_va, at_vb, at_do;
    const float *lse, *delta;
    E* dq;                 // WITH_DQ, when acc_q is null
    void *acc_k, *acc_v;   // [BH][T][D] gradients of the rows: fixed point (long long) or float
    void* acc_q;           // WITH_DQ: when non-null, dQ / alpha is added here instead of being written to dq
    int acc_q_rows;        // 0: acc_q is [BH][T][D]; else it holds the first acc_q_rows queries only, [BH][rows][D]
    // when non-null, LSE and Delta of query tile 0 come from the partials the split STATS launch left here
    const float* stats_part;
    int split_rounds;      // tile 0 only: rounds dealt out to workgroups (see tdp_f32_tile0_kernel), else 0
    // tdp_f32_bwd_kernel: workgroups per query tile (blockIdx.z); workgroup z walks rounds m_lo + z, m_lo + z + parts, ...
    // More than one needs acc_q where dQ is produced (each workgroup holds a share of it)
    int round_parts;
    // fixed-point accumulators (common.hpp); scale_parts null: the accumulators are float
    const unsigned* scale_parts;
    unsigned* poison;
    int scale_bias;
    unsigned bit_k, bit_v;  // poison bits of acc_k / acc_v
    int T, BH, nqt;        // nqt: query tiles this launch covers (tiles 0 .. nqt - 1)
    float alpha;
    TdpMask mask;
};

__device__ __forceinline__ float half_sum(float v) {  // over the 32 lanes of a wave half
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// `only_round` >= 0: this workgroup walks that round of rows only; else every `parts`-th round from the `part`-th on.
// `bx` >= 0: the workgroup's place in a grid of its own (a kernel that runs these workgroups beside others passes it);
// else blockIdx.x, and blockIdx.y picks the gradient columns
template <typename E, int D, int DOUT, bool WITH_DQ>
__device__ __forceinline__ void f32_bwd_body(const F32BwdParams<E>& p, int only_round, int part = 0, int parts = 1,
                                             int bx = -1) {
    constexpr int DTO = DOUT / 32, KS = D / 2, LD = D + 1, NW = kF32Waves;
    // form the B operands of the score products as they are used (two LDS reads and a multiply per MFMA) instead of
    // holding D / 2 of each in registers where the accumulators leave no room for them: both at D = 128, those of
    // dP alone at D = 64 in the launch that also carries the dQ accumulators
    constexpr bool FLY = D > 64, FLY_G = FLY || (D == 64 && WITH_DQ);
    // dQ of the tile, summed over the rounds: in registers up to 64 columns; beyond that the accumulators of a round
    // leave no room for it and it lives in LDS, where the waves add their round's share one after another
    constexpr bool DQ_LDS = WITH_DQ && DOUT > 64;
    extern __shared__ __align__(16) float smem_f[];
    float* sK = smem_f;                 // [2][32][LD]
    float* sV = sK + 2 * 32 * LD;       // [2][32][LD]
    float* sQ = sV + 2 * 32 * LD;       // [32][LD]  Q * alpha * log2(e)
    float* sDO = sQ + 32 * LD;          // [32][LD]
    float* sKb = sDO + 32 * LD;         // [NW][D]
    float* sVb = sKb + NW * D;          // [NW][D]
    float* sO = DQ_LDS ? sVb + NW * D : sK;  // [DOUT][33]  dQ of the tile (aliases the stages when it is only formed at the end)

    int bh, order;
    const int block_x = bx < 0 ? (int)blockIdx.x : bx;
    if (!xcd_tile(p.BH, p.nqt, block_x >> 3, block_x & 7, bh, order)) return;
    const int qt = p.nqt - 1 - order;
    const int c0 = (bx < 0 ? (int)blockIdx.y : 0) * DOUT;  // first gradient column of this workgroup

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D;
    const int b_ = bh / p.H, h_ = bh % p.H;
    auto slice = [&](const E* t, const TensorAt& at) { return t + (size_t)b_ * at.sb + (size_t)h_ * at.sh; };
    const E* __restrict__ KA = slice(p.ka, p.at_ka);
    const E* __restrict__ VA = slice(p.va, p.at_va);
    const E* __restrict__ KB = slice(p.kb, p.at_kb);
    const E* __restrict__ VB = slice(p.vb, p.at_vb);
    const E* __restrict__ Qs = slice(p.q, p.at_q);
    const TdpMask mask = p.mask;
    const float scale_log2 = p.alpha * kLog2e;
    const float fscale = p.scale_parts ? fixed_scale_value(fixed_scale_field(p.scale_parts, bh, p.scale_bias)) : 0.f;

    const int q0 = qt * 32, q1 = min(T - 1, q0 + 31);
    const int q = q0 + n;
    const Range rows = row_range(mask, q0, q1, T);
    int m_lo = rows.lo / NW + part, m_hi = rows.hi / NW;
    if (only_round >= 0) {
        m_lo = max(m_lo, only_round);
        m_hi = min(m_hi, only_round);
    }
    if (parts > 1 && m_lo > m_hi) return;  // fewer rounds than workgroups: nothing to add (uniform, before any barrier)
    for (int idx = tid; idx < 32 * D; idx += 512) {
        const int r = idx / D, d = idx % D;
        const size_t row = (size_t)min(q0 + r, T - 1);
        sQ[r * LD + d] = (float)Qs[row * p.at_q.st + d] * scale_log2;
        sDO[r * LD + d] = (float)slice(p.d_o, p.at_do)[row * p.at_do.st + d];
    }
    // a query past the end of the sequence gets a huge LSE: its P is exactly 0
    float lse2 = 1.0e30f, delta = 0.f;
    if (q < T) {
        if (p.stats_part) {  // tile 0: join the partials of the rounds
            const float* part = p.stats_part + ((size_t)bh * 32 + n) * p.split_rounds * 3;
            float M = kNegBig, L = 0.f, num = 0.f;
            for (int z = 0; z < p.split_rounds; ++z) M = fmaxf(M, part[z * 3]);
            for (int z = 0; z < p.split_rounds; ++z) {
                const float w = fast_exp2(part[z * 3] - M);
                L += part[z * 3 + 1] * w;
                num += part[z * 3 + 2] * w;
            }
            lse2 = M + fast_log2(L);
            delta = num / L;
        } else {
            lse2 = p.lse[(size_t)bh * T + q] * kLog2e;
            delta = p.delta[(size_t)bh * T + q];
        }
    }

    f32x16 accDQ[DQ_LDS ? 1 : DTO];
#pragma unroll
    for (int dt = 0; dt < (DQ_LDS ? 1 : DTO); ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) accDQ[dt][i] = 0.f;
    if constexpr (DQ_LDS)  // the first round's opening barrier orders this before the first addition
        for (int idx = tid; idx < DOUT * 33; idx += 512) sO[idx] = 0.f;

    StageE<E, D> regs;
    for (int m = m_lo; m <= m_hi; m += parts) {
        const int b = m * NW + wave;
        const Range ra = streamed_range(mask, q0, q1, min(m * NW, T - 1), T);
        const Range rb = streamed_range(mask, q0, q1, min(m * NW + NW - 1, T - 1), T);
        const int st_lo = min(ra.lo, rb.lo) / 32, st_hi = max(ra.hi, rb.hi) / 32;
        const bool row_ok = b <= rows.hi && b >= rows.lo;
        const Range mine = streamed_range(mask, q0, q1, min(b, T - 1), T);

        __syncthreads();
        for (int idx = tid; idx < NW * D; idx += 512) {
            const int r = idx / D, d = idx % D;
            const size_t row = (size_t)min(m * NW + r, T - 1);
            sKb[idx] = (float)KB[row * p.at_kb.st + d];
            sVb[idx] = (float)VB[row * p.at_vb.st + d];
        }
        if (st_lo <= st_hi) {
            stage_fetch_e<E, D>(regs, KA, VA, st_lo * 32, T, p.at_ka.st, p.at_va.st);
            stage_store_e<E, D>(regs, sK, sV);
        }
        __syncthreads();

        float bq[FLY ? 1 : KS], bg[FLY_G ? 1 : KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            if constexpr (!FLY) bq[s] = sQ[n * LD + g * KS + s] * sKb[wave * D + g * KS + s];
            if constexpr (!FLY_G) bg[s] = sDO[n * LD + g * KS + s] * sVb[wave * D + g * KS + s];
        }
        f32x16 accQ[DTO], accT[DTO];
#pragma unroll
        for (int dt = 0; dt < DTO; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                accQ[dt][i] = 0.f;
                accT[dt][i] = 0.f;
            }

        for (int st = st_lo; st <= st_hi; ++st) {
            const int buf = (st - st_lo) & 1;
            const float* cK = sK + buf * 32 * LD;
            const float* cV = sV + buf * 32 * LD;
            const bool more = st < st_hi;
            if (more) stage_fetch_e<E, D>(regs, KA, VA, (st + 1) * 32, T, p.at_ka.st, p.at_va.st);
            const int a0 = st * 32;
            if (row_ok && a0 + 31 >= mine.lo && a0 <= mine.hi) {
                f32x16 s, dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                    dp[i] = 0.f;
                }
                // The per-lane parts of the LDS addresses, opaque to the compiler from here on: every read below is
                // then this base plus a compile-time offset (the instruction's immediate field).  Left to itself the
                // compiler computes the hundreds of addresses of the unrolled loops ahead of the loops and keeps them
                // in registers (D = 128: 150 of them spilled to scratch memory).
                int row_base = n * LD + g * KS, own_base = wave * D + g * KS, out_base = 4 * g * LD + c0 + n;
                asm volatile("" : "+v"(row_base), "+v"(out_base), "+v"(own_base));
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const float oq = FLY ? sQ[row_base + ks] * sKb[own_base + ks] : bq[FLY ? 0 : ks];
                    const float og = FLY_G ? sDO[row_base + ks] * sVb[own_base + ks] : bg[FLY_G ? 0 : ks];
                    s = mma_f32(cK[row_base + ks], oq, s);
                    dp = mma_f32(cV[row_base + ks], og, dp);
                    // keep the operand reads of later k-steps from being hoisted over these (they would have to be
                    // held in registers the accumulators need)
                    if (FLY_G && (ks & 7) == 7) __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int a = a0 + c_row(g, i);
                    const bool ok = a < T && tdp_valid(mask, q, a, b);
                    const float pv = ok ? fast_exp2(s[i] - lse2) : 0.f;
                    s[i] = pv;
                    dp[i] = pv * (dp[i] - delta);
                }
#pragma unroll
                for (int dt = 0; dt < DTO; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        // row c_row(g, i) = c_row(0, i) + 4 g
                        accT[dt] = mma_f32(cV[out_base + c_row(0, i) * LD + dt * 32], s[i], accT[dt]);
                        accQ[dt] = mma_f32(cK[out_base + c_row(0, i) * LD + dt * 32], dp[i], accQ[dt]);
                        if (FLY_G && (i & 3) == 3) __builtin_amdgcn_sched_barrier(0);
                    }
            }
            if (more) {
                stage_store_e<E, D>(regs, sK + (buf ^ 1) * 32 * LD, sV + (buf ^ 1) * 32 * LD);
                __syncthreads();
            }
        }
        if (row_ok) {
            int q_base = n * LD + c0 + 4 * g, kb_base = wave * D + c0 + 4 * g;  // opaque bases, as in the loop above
            asm volatile("" : "+v"(q_base), "+v"(kb_base));
#pragma unroll
            for (int dt = 0; dt < DTO; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int d = c0 + dt * 32 + c_row(g, i), dc = dt * 32 + c_row(0, i);
                    if constexpr (WITH_DQ && !DQ_LDS) accDQ[dt][i] += accQ[dt][i] * sKb[kb_base + dc];
                    // sQ holds Q * alpha * log2(e): alpha is wanted, log2(e) is not
                    const float rk = half_sum(accQ[dt][i] * sQ[q_base + dc]) * kLn2;
                    const float rv = half_sum(accT[dt][i] * sDO[q_base + dc]);
                    if (n == 0) {
                        const size_t idx = base + (size_t)b * D + d;
                        unsigned* prow = p.poison + (size_t)bh * T + b;
                        shared_add(p.acc_k, idx, rk, fscale, prow, p.bit_k);
                        shared_add(p.acc_v, idx, rv, fscale, prow, p.bit_v);
                    }
                }
        }
        if constexpr (DQ_LDS) {
            // dQ[q] += Yq (.) K2[b], one wave after another: a fixed summation order (every wave takes part in the
            // barriers, whether or not it had a row this round)
            for (int w = 0; w < NW; ++w) {
                if (wave == w && row_ok) {
                    int kb_base = wave * D + c0 + 4 * g, o_base = 4 * g * 33 + n;
                    asm volatile("" : "+v"(kb_base), "+v"(o_base));
#pragma unroll
                    for (int dt = 0; dt < DTO; ++dt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const int dc = dt * 32 + c_row(0, i);
                            sO[o_base + dc * 33] += accQ[dt][i] * sKb[kb_base + dc];
                        }
                }
                __syncthreads();
            }
        }
    }

    if constexpr (WITH_DQ) {
        __syncthreads();
        if constexpr (!DQ_LDS) {
            for (int idx = tid; idx < DOUT * 33; idx += 512) sO[idx] = 0.f;
            __syncthreads();
            for (int w = 0; w < NW; ++w) {  // one wave after another: a fixed summation order
                if (wave == w) {
#pragma unroll
                    for (int dt = 0; dt < DTO; ++dt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) sO[(dt * 32 + c_row(g, i)) * 33 + n] += accDQ[dt][i];
                }
                __syncthreads();
            }
        }
        for (int idx = tid; idx < 32 * DOUT; idx += 512) {
            const int r = idx / DOUT, d = idx % DOUT;
            if (q0 + r < T) {
                const size_t off = base + (size_t)(q0 + r) * D + c0 + d;
                if (p.acc_q)
                    shared_add(p.acc_q, p.acc_q_rows ? ((size_t)bh * p.acc_q_rows + q0 + r) * D + c0 + d : off,
                               sO[d * 33 + r], fscale, p.poison + (size_t)bh * T + q0 + r, kPoisonDQ);
                else
                    p.dq[off] = (E)(sO[d * 33 + r] * p.alpha);
            }
        }
    }
}

template <typename E, int D, int DOUT, bool WITH_DQ>
__global__ __launch_bounds__(512) void tdp_f32_bwd_kernel(F32BwdParams<E> p) {
    f32_bwd_body<E, D, DOUT, WITH_DQ>(p, -1, blockIdx.z, gridDim.z);
}

// Query tile 0 of a 16-bit backward, both launches' roles and all rounds at once: blockIdx.z = role * rounds + round
// (role 0: rows = (K2, V2), with dQ; role 1: rows = (K1, U)).  A tile of 32 queries has at most four rounds of
// eight rows; one workgroup walking them one after another is 4 x ~25 us of pure latency.
template <typename E, int D, int DOUT>
__device__ __forceinline__ void f32_tile0_block(const F32BwdParams<E>& r0, const F32BwdParams<E>& r1, int roles_mask, int z,
                                                int bx = -1) {
    const int role = z / r0.split_rounds, round = z % r0.split_rounds;
    if (!((roles_mask >> role) & 1)) return;
    if (role == 0) {
        if (roles_mask & 4) f32_bwd_body<E, D, DOUT, true>(r0, round, 0, 1, bx);
        else f32_bwd_body<E, D, DOUT, false>(r0, round, 0, 1, bx);
    } else {
        f32_bwd_body<E, D, DOUT, false>(r1, round, 0, 1, bx);
    }
}
template <typename E, int D, int DOUT>
__global__ __launch_bounds__(512) void tdp_f32_tile0_kernel(F32BwdParams<E> r0, F32BwdParams<E> r1, int roles_mask) {
    f32_tile0_block<E, D, DOUT>(r0, r1, roles_mask, blockIdx.z);
}

template <int D>
constexpr size_t f32_bwd_smem() {
    // stages, Q and dO, the rows of a round; D = 128: dQ of the tile (f32_bwd_body's DQ_LDS)
    return sizeof(float) * (size_t)(4 * 32 * (D + 1) + 2 * 32 * (D + 1) + 2 * kF32Waves * D + (D > 64 ? D * 33 : 0));
}

template <int D>
constexpr size_t f32_fwd_smem() {
    return sizeof(float) * (size_t)(4 * 32 * (D + 1) + 32 * (D + 1) + 2 * kF32Waves * D + 2 * kF32Waves * 32);
}


// where the six inputs lie (F32Params::H and at_*)
struct InputsAt {
    int H;
    TensorAt q, d_o, k1, u, k2, v2;
};
InputsAt dense_inputs(int T, int D) {
    const TensorAt d = dense_at(1, T, D);
    return InputsAt{1, d, d, d, d, d, d};
}
InputsAt inputs_of(const FirstTileArgs& a) {
    if (a.H <= 0) return dense_inputs(a.T, a.D);
    return InputsAt{a.H, a.at_q, a.at_do, a.at_k1, dense_at(a.H, a.T, a.D), a.at_k2, a.at_v2};
}
// streamed = (K1, U), rows = (K2, V2), or the two exchanged
template <typename P>
void place_inputs(P& p, const InputsAt& at, bool exchanged) {
    p.H = at.H; p.at_q = at.q; p.at_do = at.d_o;
    p.at_ka = exchanged ? at.k2 : at.k1; p.at_va = exchanged ? at.v2 : at.u;
    p.at_kb = exchanged ? at.k1 : at.k2; p.at_vb = exchanged ? at.u : at.v2;
}

// Query tile 0 alone, first half: launches the STATS pass (its rounds dealt out to workgroups) and fills in the
// parameters of the backward pass over the tile for both roles.  The backward workgroups themselves are
// (8 xcd_slots(BH, 1)) x (2 rounds) calls of f32_tile0_block: tdp_f32_tile0_kernel, or the tail of another grid.
template <typename E, int D>
hipError_t tile0_prepare(const FirstTileArgs& a, hipStream_t st, F32BwdParams<E>& r0, F32BwdParams<E>& r1, int& roles,
                         int& rounds) {
    rounds = (std::min(a.T, 32) + kF32Waves - 1) / kF32Waves;
    const TdpMask natural{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    const bool own_dq_acc = a.want_q && !a.acc_q;  // dQ of the tile is summed over its rounds in a.dq0_acc
    {
        F32Params<E> p{};
        p.q = (const E*)a.q; p.ka = (const E*)a.k1; p.kb = (const E*)a.k2; p.va = (const E*)a.u; p.vb = (const E*)a.v2;
        place_inputs(p, inputs_of(a), false);
        p.o = nullptr; p.lse = nullptr; p.d_o = (const E*)a.d_o; p.delta = a.delta_f32;
        p.split_rounds = rounds;
        p.zero_ptr = own_dq_acc ? (unsigned*)a.dq0_acc : nullptr;
        p.zero_words = own_dq_acc ? 32 * D * (a.scale_parts ? 2 : 1) : 0;
        p.T = a.T; p.BH = a.BH; p.nqt = 1;
        p.scale_log2 = a.alpha * kLog2e;
        p.mask = natural;
        auto kern = tdp_f32_fwd_kernel<E, D, true>;
        constexpr size_t smem = f32_fwd_smem<D>();
        if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, 1), rounds), dim3(512), smem, st, p);
    }
    r0 = F32BwdParams<E>{};
    r0.q = (const E*)a.q; r0.d_o = (const E*)a.d_o; r0.lse = nullptr; r0.delta = nullptr;
    r0.stats_part = a.delta_f32; r0.split_rounds = rounds; r0.round_parts = 1;
    r0.dq = (E*)a.dq; r0.acc_q = a.acc_q ? a.acc_q : a.dq0_acc; r0.acc_q_rows = a.acc_q ? 0 : 32;
    r0.scale_parts = a.scale_parts; r0.poison = a.poison; r0.scale_bias = a.scale_bias;
    r0.T = a.T; r0.BH = a.BH; r0.nqt = 1; r0.alpha = a.alpha;
    r1 = r0;
    r0.ka = (const E*)a.k1; r0.va = (const E*)a.u; r0.kb = (const E*)a.k2; r0.vb = (const E*)a.v2;
    place_inputs(r0, inputs_of(a), false);
    r0.acc_k = a.acc_k2; r0.acc_v = a.acc_v2; r0.bit_k = kPoisonDK2; r0.bit_v = kPoisonDV2; r0.mask = natural;
    r1.ka = (const E*)a.k2; r1.va = (const E*)a.v2; r1.kb = (const E*)a.k1; r1.vb = (const E*)a.u;
    place_inputs(r1, inputs_of(a), true);
    r1.acc_k = a.acc_k1; r1.acc_v = a.acc_u; r1.bit_k = kPoisonDK1; r1.bit_v = kPoisonDU;
    r1.mask = TdpMask{natural.causal, natural.wb, natural.wa, natural.rab, natural.lab};
    roles = ((a.want_q || a.want_k2) ? 1 : 0) | (a.want_k1 ? 2 : 0) | (a.want_q ? 4 : 0);
    return hipGetLastError();
}

}  // namespace
}  // namespace tritt
