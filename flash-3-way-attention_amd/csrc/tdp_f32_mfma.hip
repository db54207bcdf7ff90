// Triple-dot-product trittention in true fp32 on the matrix cores (v_mfma_f32_32x32x2_f32), D = 32, 64 or 128,
// every mask.  This is the path of fp32 tensors: fp32 operands, fp32 products, fp32 accumulation (the 1e-4
// relative bar), at the fp32 matrix rate (157 TFLOP/s peak) instead of the fp32 vector rate of the VALU kernels.
//
// All tensors here are fp32 [BH, T, D]; U = SiLU(V1) (see capi.hip).
//
// Formulation (the same virtual-query one as the 16-bit kernels).  A workgroup owns 32 consecutive queries;
// its eight waves take eight consecutive rows b per round (one per wave; b = k, the K2 / V2 row, in the
// natural orientation) and sweep the streamed index a (= j, K1 / U rows) in 32-row stages shared through LDS.
// For a fixed row b the scores of the 32 queries against 32 streamed rows are one 32x32 tile
//   S^T[a, q] = sum_d KA[a, d] * (scale * Q[q, d] * KB[b, d])
// i.e. D / 2 MFMAs (K = 2 each).  The tile leaves the MFMA with lane <-> query and registers <-> streamed rows,
// which is exactly the B-operand layout of the next product
//   Tv^T[d, q] += sum_a VA^T[d, a] * P^T[a, q]
// so P is never moved between lanes, and every per-query quantity (running maximum, row sum, the merge of a
// finished row b into the output, O^T[d, q] += Tv^T[d, q] * VB[b, d]) is lane-local.
// With 64-cycle MFMAs the kernels are bound by the matrix pipe; the element-wise work (mask predicate on every
// element, online softmax) hides under it, so there is one loop body for every mask.
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

// `only_round` >= 0: this workgroup walks that round of rows only; else every `parts`-th round from the `part`-th on
template <typename E, int D, int DOUT, bool WITH_DQ>
__device__ __forceinline__ void f32_bwd_body(const F32BwdParams<E>& p, int only_round, int part = 0, int parts = 1) {
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
    if (!xcd_tile(p.BH, p.nqt, blockIdx.x >> 3, blockIdx.x & 7, bh, order)) return;
    const int qt = p.nqt - 1 - order;
    const int c0 = blockIdx.y * DOUT;  // first gradient column of this workgroup

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
__global__ __launch_bounds__(512) void tdp_f32_tile0_kernel(F32BwdParams<E> r0, F32BwdParams<E> r1, int roles_mask) {
    const int role = blockIdx.z / r0.split_rounds, round = blockIdx.z % r0.split_rounds;
    if (!((roles_mask >> role) & 1)) return;
    if (role == 0) {
        if (roles_mask & 4) f32_bwd_body<E, D, DOUT, true>(r0, round);
        else f32_bwd_body<E, D, DOUT, false>(r0, round);
    } else {
        f32_bwd_body<E, D, DOUT, false>(r1, round);
    }
}

__global__ __launch_bounds__(256) void f32_zero_kernel(long long* __restrict__ a, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) a[i] = 0;
}
// the partial maxima of |dO| that fix the scale of a slice's accumulators: grid (kScaleParts, BH)
__global__ __launch_bounds__(256) void f32_scale_kernel(const float* __restrict__ d_o, unsigned* __restrict__ parts,
                                                        size_t per_slice) {
    __shared__ unsigned red[4];
    const size_t pieces = per_slice / 4, per_part = (pieces + kScaleParts - 1) / kScaleParts;
    const size_t lo = min(pieces, blockIdx.x * per_part), hi = min(pieces, lo + per_part);
    const unsigned m = block_absmax_bits<float>(d_o + blockIdx.y * per_slice + lo * 4, hi - lo, red);
    if (threadIdx.x == 0) parts[blockIdx.y * kScaleParts + blockIdx.x] = m;
}
// fixed point -> fp32, one tensor (dQ / alpha accumulated over the workgroups of a tile)
__global__ __launch_bounds__(256) void f32_finish_q_kernel(const long long* __restrict__ acc, float* __restrict__ dq, size_t n,
                                                           int T, int D, const unsigned* __restrict__ scale_parts,
                                                           const unsigned* __restrict__ poison, float alpha) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t row = i / D;
        const double inv = fixed_scale_inverse(fixed_scale_field<false>(scale_parts, (int)(row / T), kF32FixedBias));
        dq[i] = (poison[row] & kPoisonDQ) ? __builtin_nanf("") : (float)((double)acc[i] * inv) * alpha;
    }
}
// fixed point -> fp32
__global__ __launch_bounds__(256) void f32_finish_kernel(const long long* __restrict__ acc, float* __restrict__ dk_rows,
                                                         float* __restrict__ dv_rows, size_t n, int T, int D,
                                                         const unsigned* __restrict__ scale_parts,
                                                         const unsigned* __restrict__ poison, unsigned bit_k,
                                                         unsigned bit_v) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const size_t row = i / D;
        const double inv = fixed_scale_inverse(fixed_scale_field<false>(scale_parts, (int)(row / T), kF32FixedBias));
        const unsigned bad = poison[row];
        dk_rows[i] = (bad & bit_k) ? __builtin_nanf("") : (float)((double)acc[i] * inv);
        dv_rows[i] = (bad & bit_v) ? __builtin_nanf("") : (float)((double)acc[n + i] * inv);
    }
}

template <int D>
constexpr size_t f32_bwd_smem() {
    // stages, Q and dO, the rows of a round; D = 128: dQ of the tile (f32_bwd_body's DQ_LDS)
    return sizeof(float) * (size_t)(4 * 32 * (D + 1) + 2 * 32 * (D + 1) + 2 * kF32Waves * D + (D > 64 ? D * 33 : 0));
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

// both launches of the backward over query tiles 0 .. nqt - 1
template <typename E, int D>
hipError_t launch_f32_bwd_tiles(F32BwdParams<E> p, const E* k1, const E* u, const E* k2, const E* v2, void* acc_k2,
                                void* acc_v2, void* acc_k1, void* acc_u, const TdpMask& natural, bool want_q,
                                bool want_k2, bool want_k1, hipStream_t st, const InputsAt& at) {
    // a workgroup holds all D gradient columns and forms S and dP once (D = 128: dQ's running sum is kept in LDS)
    constexpr int DOUT = D, DOUT_NODQ = D;
    auto kern_dq = tdp_f32_bwd_kernel<E, D, DOUT, true>;
    auto kern_nodq = tdp_f32_bwd_kernel<E, D, DOUT_NODQ, false>;
    constexpr size_t smem = f32_bwd_smem<D>();
    static_assert(DOUT * 33 <= 4 * 32 * (D + 1), "dQ of the tile aliases the stage buffers (D <= 64)");
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern_dq), smem); e != hipSuccess) return e;
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern_nodq), smem); e != hipSuccess) return e;
    // small grids: the rounds of a tile dealt out to several workgroups (the launch with dQ only when dQ has an accumulator)
    const int parts = std::max(1, p.round_parts);
    const dim3 grid(8 * xcd_slots(p.BH, p.nqt), D / DOUT, p.acc_q ? parts : 1), grid_nodq(8 * xcd_slots(p.BH, p.nqt), D / DOUT_NODQ, parts);
    // rows = (K2, V2), streamed = (K1, U): dQ, dK2, dV2
    p.ka = k1; p.va = u; p.kb = k2; p.vb = v2;
    place_inputs(p, at, false);
    p.acc_k = acc_k2; p.acc_v = acc_v2; p.bit_k = kPoisonDK2; p.bit_v = kPoisonDV2;
    p.mask = natural;
    if (want_q) hipLaunchKernelGGL(kern_dq, grid, dim3(512), smem, st, p);
    else if (want_k2) hipLaunchKernelGGL(kern_nodq, grid_nodq, dim3(512), smem, st, p);
    // rows = (K1, U), streamed = (K2, V2): dK1, dU (the mask with the two key indices exchanged)
    p.ka = k2; p.va = v2; p.kb = k1; p.vb = u;
    place_inputs(p, at, true);
    p.acc_k = acc_k1; p.acc_v = acc_u; p.bit_k = kPoisonDK1; p.bit_v = kPoisonDU;
    p.mask = TdpMask{natural.causal, natural.wb, natural.wa, natural.rab, natural.lab};
    if (want_k1) hipLaunchKernelGGL(kern_nodq, grid_nodq, dim3(512), smem, st, p);
    return hipGetLastError();
}

template <int D>
hipError_t launch_f32_bwd(const GenericTdpArgs& a, long long* acc, hipStream_t st) {
    const size_t n = (size_t)a.BH * a.T * D;
    const bool want_q = a.dq != nullptr, want_k2 = a.dk2 && a.dv2, want_k1 = a.dk1 && a.du;
    F32BwdParams<float> p{};
    p.q = a.q; p.d_o = a.d_o; p.lse = a.lse_in; p.delta = a.delta;
    p.round_parts = f32_round_parts(a.BH, a.T);
    const bool q_shared = want_q && p.round_parts > 1;
    p.dq = a.dq; p.acc_q = q_shared ? acc + 4 * n : nullptr; p.acc_q_rows = 0; p.stats_part = nullptr; p.split_rounds = 0;
    // scratch: four accumulators (five when the rounds of a tile are dealt out: dQ then has one too), the rows'
    // poison words, the slices' scale partials
    const size_t nacc = (p.round_parts > 1 ? 5 : 4) * n;
    const size_t rows = (size_t)a.BH * a.T, zero_n = nacc + (rows + 3) / 4 * 2;  // 16-byte aligned parts
    unsigned* poison = reinterpret_cast<unsigned*>(acc + nacc);
    unsigned* parts = reinterpret_cast<unsigned*>(acc + zero_n);
    p.scale_parts = parts; p.poison = poison; p.scale_bias = kF32FixedBias;
    p.T = a.T; p.BH = a.BH; p.nqt = (a.T + 31) / 32;
    p.alpha = a.alpha;
    size_t gz = (zero_n + 255) / 256;
    if (gz > 8192) gz = 8192;
    hipLaunchKernelGGL(f32_zero_kernel, dim3((unsigned)gz), dim3(256), 0, st, acc, zero_n);
    hipLaunchKernelGGL(f32_scale_kernel, dim3(kScaleParts, a.BH), dim3(256), 0, st, a.d_o, parts, (size_t)a.T * D);
    const TdpMask natural{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    if (hipError_t e = launch_f32_bwd_tiles<float, D>(p, a.k1, a.u, a.k2, a.v2, acc, acc + n, acc + 2 * n, acc + 3 * n,
                                                      natural, want_q, want_k2, want_k1, st, dense_inputs(a.T, D));
        e != hipSuccess)
        return e;
    size_t gf = (n + 255) / 256;
    if (gf > 4096) gf = 4096;
    if (q_shared)
        hipLaunchKernelGGL(f32_finish_q_kernel, dim3((unsigned)gf), dim3(256), 0, st, acc + 4 * n, a.dq, n, a.T, D, parts,
                           poison, a.alpha);
    if (want_k2)
        hipLaunchKernelGGL(f32_finish_kernel, dim3((unsigned)gf), dim3(256), 0, st, acc, a.dk2, a.dv2, n, a.T, D, parts,
                           poison, kPoisonDK2, kPoisonDV2);
    if (want_k1)
        hipLaunchKernelGGL(f32_finish_kernel, dim3((unsigned)gf), dim3(256), 0, st, acc + 2 * n, a.dk1, a.du, n, a.T, D,
                           parts, poison, kPoisonDK1, kPoisonDU);
    return hipGetLastError();
}

template <int D>
constexpr size_t f32_fwd_smem() {
    return sizeof(float) * (size_t)(4 * 32 * (D + 1) + 32 * (D + 1) + 2 * kF32Waves * D + 2 * kF32Waves * 32);
}

template <int D>
hipError_t launch_f32_fwd(const GenericTdpArgs& a, hipStream_t st) {
    F32Params<float> p{};
    p.q = a.q; p.ka = a.k1; p.kb = a.k2; p.va = a.u; p.vb = a.v2;
    place_inputs(p, dense_inputs(a.T, D), false);
    p.o = a.o; p.lse = a.lse;
    p.d_o = nullptr; p.delta = nullptr; p.split_rounds = 0; p.zero_ptr = nullptr; p.zero_words = 0;
    p.T = a.T; p.BH = a.BH; p.nqt = (a.T + 31) / 32;
    p.scale_log2 = a.alpha * kLog2e;
    p.mask = TdpMask{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    auto kern = tdp_f32_fwd_kernel<float, D, false>;
    constexpr size_t smem = f32_fwd_smem<D>();
    static_assert(D * 33 <= 4 * 32 * (D + 1), "the merged output aliases the stage buffers");
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, p.nqt)), dim3(512), smem, st, p);
    return hipGetLastError();
}

}  // namespace

bool f32_mfma_tdp_supported(int D) { return D == 32 || D == 64 || D == 128; }

// Measured at D = 64 with narrow windows (seven rounds of two or three stages per tile): a round costs about 25 us and
// a workgroup about 50 us before its first one, so dealing rounds out pays while the tiles alone leave more than half
// of the compute units idle (32 tiles: 245 -> 75 us per launch), and not beyond (128 tiles: 245 -> 260 us).
int f32_round_parts(int BH, int T) {
    const int tiles = BH * ((T + 31) / 32);
    return tiles >= 128 ? 1 : std::min(16, (256 + tiles - 1) / tiles);
}

// The first query tiles of a 16-bit backward, in fp32 (see the comment above tdp_f32_bwd_kernel).
template <typename E, int D>
static hipError_t launch_stats(const FirstTileArgs& a, hipStream_t st) {
    F32Params<E> p{};
    p.q = (const E*)a.q; p.ka = (const E*)a.k1; p.kb = (const E*)a.k2; p.va = (const E*)a.u; p.vb = (const E*)a.v2;
    place_inputs(p, inputs_of(a), false);
    p.o = nullptr; p.lse = a.lse_f32; p.d_o = (const E*)a.d_o; p.delta = a.delta_f32;
    p.split_rounds = 0; p.zero_ptr = nullptr; p.zero_words = 0;
    p.T = a.T; p.BH = a.BH; p.nqt = a.tiles;
    p.scale_log2 = a.alpha * kLog2e;
    p.mask = TdpMask{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    auto kern = tdp_f32_fwd_kernel<E, D, true>;
    constexpr size_t smem = f32_fwd_smem<D>();
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, p.nqt)), dim3(512), smem, st, p);
    return hipGetLastError();
}

// Query tile 0 alone: the STATS pass and the backward pass, each with its rounds dealt out to workgroups.
template <typename E, int D>
static hipError_t launch_tile0_split(const FirstTileArgs& a, hipStream_t st) {
    constexpr int DOUT = D > 64 ? 64 : D;
    const int rounds = (std::min(a.T, 32) + kF32Waves - 1) / kF32Waves;
    const int groups = (a.BH + 7) / 8;
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
    F32BwdParams<E> r0{};
    r0.q = (const E*)a.q; r0.d_o = (const E*)a.d_o; r0.lse = nullptr; r0.delta = nullptr;
    r0.stats_part = a.delta_f32; r0.split_rounds = rounds; r0.round_parts = 1;
    r0.dq = (E*)a.dq; r0.acc_q = a.acc_q ? a.acc_q : a.dq0_acc; r0.acc_q_rows = a.acc_q ? 0 : 32;
    r0.scale_parts = a.scale_parts; r0.poison = a.poison; r0.scale_bias = a.scale_bias;
    r0.T = a.T; r0.BH = a.BH; r0.nqt = 1; r0.alpha = a.alpha;
    F32BwdParams<E> r1 = r0;
    r0.ka = (const E*)a.k1; r0.va = (const E*)a.u; r0.kb = (const E*)a.k2; r0.vb = (const E*)a.v2;
    place_inputs(r0, inputs_of(a), false);
    r0.acc_k = a.acc_k2; r0.acc_v = a.acc_v2; r0.bit_k = kPoisonDK2; r0.bit_v = kPoisonDV2; r0.mask = natural;
    r1.ka = (const E*)a.k2; r1.va = (const E*)a.v2; r1.kb = (const E*)a.k1; r1.vb = (const E*)a.u;
    place_inputs(r1, inputs_of(a), true);
    r1.acc_k = a.acc_k1; r1.acc_v = a.acc_u; r1.bit_k = kPoisonDK1; r1.bit_v = kPoisonDU;
    r1.mask = TdpMask{natural.causal, natural.wb, natural.wa, natural.rab, natural.lab};
    const int roles = ((a.want_q || a.want_k2) ? 1 : 0) | (a.want_k1 ? 2 : 0) | (a.want_q ? 4 : 0);
    auto kern = tdp_f32_tile0_kernel<E, D, DOUT>;
    constexpr size_t smem = f32_bwd_smem<D>();
    if (hipError_t e = ensure_dynamic_smem(reinterpret_cast<const void*>(kern), smem); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(8 * xcd_slots(a.BH, 1), D / DOUT, 2 * rounds), dim3(512), smem, st, r0, r1, roles);
    return hipGetLastError();
}

template <typename E>
static hipError_t first_tile_typed(const FirstTileArgs& a, hipStream_t st) {
    if (a.tiles == 1) {
        return a.D == 32 ? launch_tile0_split<E, 32>(a, st) : a.D == 64 ? launch_tile0_split<E, 64>(a, st)
             : a.D == 128 ? launch_tile0_split<E, 128>(a, st) : hipErrorInvalidValue;
    }
    // the rows' log-sum-exp and Delta once more, in fp32 from the same tensors: the saved LSE carries the 16-bit
    // rounding of the forward's scores and Delta that of the stored output, and nearly one-hot rows show both
    hipError_t es = a.D == 32 ? launch_stats<E, 32>(a, st) : a.D == 64 ? launch_stats<E, 64>(a, st)
                  : a.D == 128 ? launch_stats<E, 128>(a, st) : hipErrorInvalidValue;
    if (es != hipSuccess) return es;
    F32BwdParams<E> p{};
    p.q = (const E*)a.q; p.d_o = (const E*)a.d_o; p.lse = a.lse_f32; p.delta = a.delta_f32;
    p.dq = (E*)a.dq; p.acc_q = a.acc_q; p.acc_q_rows = 0; p.stats_part = nullptr; p.split_rounds = 0;
    p.round_parts = a.round_parts;
    p.scale_parts = a.scale_parts; p.poison = a.poison; p.scale_bias = a.scale_bias;
    p.T = a.T; p.BH = a.BH; p.nqt = a.tiles;
    p.alpha = a.alpha;
    const TdpMask natural{a.causal, a.k1_window, a.k2_window, a.kk_left, a.kk_right};
    const E *k1 = (const E*)a.k1, *u = (const E*)a.u, *k2 = (const E*)a.k2, *v2 = (const E*)a.v2;
    const bool wq = a.want_q, wk2 = a.want_k2, wk1 = a.want_k1;
    if (a.D == 32)
        return launch_f32_bwd_tiles<E, 32>(p, k1, u, k2, v2, a.acc_k2, a.acc_v2, a.acc_k1, a.acc_u, natural, wq, wk2, wk1, st, inputs_of(a));
    if (a.D == 64)
        return launch_f32_bwd_tiles<E, 64>(p, k1, u, k2, v2, a.acc_k2, a.acc_v2, a.acc_k1, a.acc_u, natural, wq, wk2, wk1, st, inputs_of(a));
    if (a.D == 128)
        return launch_f32_bwd_tiles<E, 128>(p, k1, u, k2, v2, a.acc_k2, a.acc_v2, a.acc_k1, a.acc_u, natural, wq, wk2, wk1, st, inputs_of(a));
    return hipErrorInvalidValue;
}
hipError_t f32_mfma_tdp_bwd_first_tile(const FirstTileArgs& a, hipStream_t st) {
    return a.is_bf16 ? first_tile_typed<__bf16>(a, st) : first_tile_typed<_Float16>(a, st);
}

hipError_t f32_mfma_tdp_fwd(const GenericTdpArgs& a, hipStream_t st) {
    if (a.D == 32) return launch_f32_fwd<32>(a, st);
    if (a.D == 64) return launch_f32_fwd<64>(a, st);
    if (a.D == 128) return launch_f32_fwd<128>(a, st);
    return hipErrorInvalidValue;
}

size_t f32_mfma_tdp_bwd_scratch_elems(int BH, int T, int D) {
    return (f32_round_parts(BH, T) > 1 ? 5 : 4) * (size_t)BH * T * D + ((size_t)BH * T + 3) / 4 * 2 +
           (size_t)BH * kScaleParts / 2;
}

hipError_t f32_mfma_tdp_bwd(const GenericTdpArgs& a, long long* scratch, hipStream_t st) {
    if (a.D == 32) return launch_f32_bwd<32>(a, scratch, st);
    if (a.D == 64) return launch_f32_bwd<64>(a, scratch, st);
    if (a.D == 128) return launch_f32_bwd<128>(a, scratch, st);
    return hipErrorInvalidValue;
}

}  // namespace tritt
