// Dot-product-sum trittention on MFMA (gfx950) for 16-bit tensors, D = 64 or 128.
//
// The score separates,  exp(alpha (Q_q.K2_t + K1_s.K2_t)) = exp(alpha Q_q.K2_t) exp(alpha K1_s.K2_t),
// and the mask (s <= t <= q, t - s <= k_diff) never couples s with q, so the op is two chained
// banded attentions (O(T^2 D) instead of O(T^3 D)):
//   inner:  lse1[t] = logsumexp_s alpha K1_s.K2_t,  R[t] = softmax_s(.) @ U,  W[t] = R[t] * V2[t]
//   outer:  O[q] = softmax_t(alpha Q_q.K2_t + lse1[t]) @ W,  LSE[q] = logsumexp_t(.)
// and the backward is the two attention backwards chained through (dR, dlse1).
//
// Three kernels, each a generic "attention with a per-key bias" building block on 32x32x16 MFMA:
//   attn_fwd_mfma_kernel       owner = 32 query-like rows;  out, out*mul, (out*mul)^T, lse
//   attn_bwd_row_mfma_kernel   owner = 32 query-like rows;  dX
//   attn_bwd_col_mfma_kernel   owner = 32 key-like rows;    dK, dV, dbias (+ the element-wise link
//                              between the two passes when it runs the outer pass)
// A workgroup is kW (2 or 4) waves that share one owner tile and split the streamed 32-row tiles between
// them round-robin (their partial results meet in LDS).
// Every tile is computed transposed where needed so that the owner index sits on the MFMA column
// (= lane) axis: softmax statistics, LSE and Delta stay lane-local, and with the permuted row order
// of mfma.hpp the probabilities leave one MFMA in exactly the operand layout of the next.
// Streamed operands are read straight from global memory, 16 B per lane, from operand-packed
// copies: the 64 x 16 B that one MFMA operand load needs are one contiguous kilobyte (a gather of
// 16-byte pieces from 32 different rows costs one cache-line lookup per row, and that address
// traffic, not MFMA or bandwidth, was what bound these kernels).  Two packings of a [T][D] tensor,
// both in tiles of 32 rows and both exactly Tp x D elements:
//   P1 (k-slots run along d; rows permuted by key_of_row):  [tile][ks][lane][8]
//   P2 (k-slots run along the row index; "transposed use"): [tile][dt][kk][lane][8]
// The prep kernel writes them for the inputs, the producing epilogues for W and dR.  Every output
// element has one owner: no atomics, bitwise reproducible.
#include "kernels.hpp"
#include "mfma.hpp"
#include "direct_lds.hpp"

namespace tritt {
namespace {

constexpr int kLdr = 33;  // LDS row stride (floats) of the cross-wave reduction tiles
constexpr float kLazyRaise = 8.0f;  // log2 units a score may exceed the running reference before it is raised

// MFMA row that holds key offset k of a 32-key tile (inverse of key_of_row)
__device__ __forceinline__ int row_of_key(int k) {
    const int i = 8 * (k >> 4) + (k & 7), g = (k >> 3) & 1;
    return ((i >> 2) << 3) | (g << 2) | (i & 3);
}
// XCD-aware block order of a 1-D grid of 8 * xcd_slots(BH, ntiles) workgroups (common.hpp): every XCD gets its own
// (batch, head) slices and their packed operands stay in that XCD's L2.  `tile` counts 0 .. ntiles-1 in launch order.
// False: a padding block.
__device__ __forceinline__ bool block_to_tile(int BH, int ntiles, int& bh, int& tile) {
    return xcd_tile(BH, ntiles, blockIdx.x >> 3, blockIdx.x & 7, bh, tile);
}
// owner tiles a launch of the attention kernels hands out (paired: a long and a short one per workgroup)
__device__ __forceinline__ int launch_tiles(int pair, int nt) { return pair ? (nt + 1) / 2 : nt; }

// Under a full causal mask the owner tiles of a launch are a triangle: the longest walks nt streamed tiles, the
// shortest one, and with one tile per workgroup the launch lasts as long as its longest tile while most SIMDs
// idle.  Paired, a workgroup takes tile `tile` and then tile nt - 1 - tile of the launch order: nt + 1 streamed
// tiles for every workgroup.  Returns how many owner tiles this workgroup walks; `part` selects one.
__device__ __forceinline__ int owner_tiles(int pair, int nt, int tile) { return (pair && tile != nt - 1 - tile) ? 2 : 1; }
__device__ __forceinline__ int owner_tile(int nt, int tile, int part) { return part ? nt - 1 - tile : tile; }

// element offsets of (row, d) in the two packings
template <int D>
__device__ __forceinline__ size_t p1_index(int row, int d) {
    return ((size_t)((row >> 5) * (D / 16) + (d >> 4)) * 64 + ((d >> 3) & 1) * 32 + row_of_key(row & 31)) * 8 + (d & 7);
}
template <int D>
__device__ __forceinline__ size_t p2_index(int row, int d) {
    const int a = row & 31;
    return ((size_t)(((row >> 5) * (D / 32) + (d >> 5)) * 2 + (a >> 4)) * 64 + ((a >> 3) & 1) * 32 + (d & 31)) * 8 + (a & 7);
}
// the operand loads: lane's 16 bytes of (tile t, k-step ks) / (tile t, d-tile dt, half kk)
template <typename E, int D>
__device__ __forceinline__ const E* p1_at(const E* z, int t, int ks, int lane) {
    return z + ((size_t)(t * (D / 16) + ks) * 64 + lane) * 8;
}
template <typename E, int D>
__device__ __forceinline__ const E* p2_at(const E* z, int t, int dt, int kk, int lane) {
    return z + ((size_t)((t * (D / 32) + dt) * 2 + kk) * 64 + lane) * 8;
}

template <typename E>
__device__ __forceinline__ typename Mma<E>::v8 ld8(const E* p) {
    return *reinterpret_cast<const typename Mma<E>::v8*>(p);
}

// 16 fp32 values of one lane (registers of a C tile) -> the two 8-wide 16-bit operands they form
template <typename E>
__device__ __forceinline__ void pack16(const float (&x)[16], typename Mma<E>::v8 (&out)[2]) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const typename Mma<E>::v2 t = Mma<E>::pack(x[8 * h + e], x[8 * h + e + 1]);
            out[h][e] = t[0];
            out[h][e + 1] = t[1];
        }
}

// 16 floats of a lane from a 32-float vector in LDS: element i is the value of key / row key_of(g, i)
__device__ __forceinline__ void tile_vector(const float* sv, int g, float (&out)[16]) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const float4 v = *reinterpret_cast<const float4*>(sv + 16 * h + 8 * g + 4 * c);
            out[8 * h + 4 * c] = v.x; out[8 * h + 4 * c + 1] = v.y; out[8 * h + 4 * c + 2] = v.z; out[8 * h + 4 * c + 3] = v.w;
        }
}

// pair (query-like row r, key-like row a) takes part
__device__ __forceinline__ bool pair_ok(int T, int causal, int k_diff, int r, int a) {
    return (r < T) & (a < T) & ((!causal) | ((a <= r) & (r - a <= k_diff)));
}

// A [B,H,T,D] tensor where it lies.  SV (strided views): element (b, h, t, d) at b sb + h sh + t st + d, the caller's
// strides for the caller's tensors and dense ones for the workspace's own row-major tensors; slices are indexed
// (batch, head).  Otherwise every tensor is dense [BH][T][D], the slice index is bh alone and the row pitch is the
// compile-time D (the strided form costs the dense calls 2-4 % at B=4 H=8 T=1024, so they keep their own kernels).
template <typename E, bool SV>
struct View;
template <typename E>
struct View<E, true> {
    const E* p;
    long long sb, sh;
    unsigned st;
    __device__ __forceinline__ const E* row(int2 at, int r, int, int) const {
        return p + (size_t)at.x * sb + (size_t)at.y * sh + (size_t)(unsigned)r * st;
    }
    __device__ __forceinline__ explicit operator bool() const { return p != nullptr; }
};
template <typename E>
struct View<E, false> {
    const E* p;
    __device__ __forceinline__ const E* row(int2 at, int r, int T, int D) const { return p + ((size_t)at.x * T + r) * D; }
    __device__ __forceinline__ explicit operator bool() const { return p != nullptr; }
};
// the slice's index in the views' terms: (batch, head), or (bh, -) for dense tensors
template <bool SV>
__device__ __forceinline__ int2 slice_at(int bh, int H) {
    return SV ? make_int2(bh / H, bh % H) : make_int2(bh, 0);
}

template <int D>
__device__ __forceinline__ void spill_tiles(float* sO, int wave, const f32x16 (&acc)[D / 32], int n, int g) {
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sO[(wave * D + 32 * dt + c_row(g, i)) * kLdr + n] = acc[dt][i];
}

// ------------------------------------------------------------------------------------ forward
template <typename E, bool SV>
struct AttnFwdP {
    View<E, SV> x;      // query-like rows
    const E* kp;        // [BH][Tp*D]   key-like rows, packing P1
    const E* vp2;       // [BH][Tp*D]   values, packing P2
    const float* bias;  // [BH][Tp] per-key bias in log2 units, or null
    View<E, SV> mul;    // or null
    E* out;             // [BH][T][D] or null
    float* out_f32;     // [BH][T][D] or null
    E* outm;            // out * mul, [BH][T][D] or null
    E* outm_p1;         // out * mul, packing P1, or null
    E* outm_p2;         // out * mul, packing P2, or null
    float* lse;         // [BH][lse_stride]
    int lse_stride;
    int BH;
    int H;              // heads per batch entry in the views' indexing
    float lse_scale;    // lse = lse_scale * log2-sum-exp2
    int T, Tp;
    float scale_log2;
    int causal, k_diff;
    int pair;           // a workgroup takes two owner tiles, a long and a short one (see owner_tiles)
};

// kW: waves per workgroup (they split the streamed tiles of one owner tile).
// Two waves per SIMD are asked for wherever the kernel fits 256 registers: a workgroup of 128 or 256 threads alone
// would let the compiler plan for 512, and it then keeps every MFMA result in accumulation registers and copies the
// accumulators to and from vector registers around the rescaling, every tile (80 of 240 vector instructions).
template <typename E, int D, int kW, bool SV>
__global__ __launch_bounds__(64 * kW, 2) void attn_fwd_mfma_kernel(AttnFwdP<E, SV> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    constexpr int KS = D / 16, DT = D / 32;
    extern __shared__ __align__(16) char smem_raw[];
    float* sO = reinterpret_cast<float*>(smem_raw);  // [kW][D][kLdr]
    float* sM = sO + kW * D * kLdr;                  // [kW][32]
    float* sL = sM + kW * 32;                        // [kW][32]

    int bh, tile0;
    if (!block_to_tile(p.BH, launch_tiles(p.pair, p.Tp / 32), bh, tile0)) return;
    const int nparts = owner_tiles(p.pair, p.Tp / 32, tile0);
    for (int op = 0; op < nparts; ++op) {
    if (op) __syncthreads();  // the merge tiles of the first owner tile have been read
    const int tile = owner_tile(p.Tp / 32, tile0, op);
    const int r0 = (p.Tp / 32 - 1 - tile) * 32;  // longest rows first
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T, Tp = p.Tp;
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp, vb = (size_t)bh * Tp;
    const E* __restrict__ KP = p.kp + tb;
    const E* __restrict__ VP2 = p.vp2 + tb;
    const float* __restrict__ bias = p.bias ? p.bias + vb : nullptr;
    const int r = r0 + n;
    const int2 at = slice_at<SV>(bh, p.H);
    const E* __restrict__ xrow = p.x.row(at, min(r, T - 1), T, D);

    v8 xb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xb[ks] = ld8<E>(xrow + 16 * ks + 8 * g);

    const int a_lo = p.causal ? max(0, r0 - p.k_diff) : 0;
    const int a_hi = p.causal ? min(T - 1, r0 + 31) : T - 1;
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    // Operands of a streamed tile are fetched one tile ahead, into the registers the previous tile has
    // just consumed (each wave runs only a handful of tiles, so two dependent global round trips per
    // tile would be most of its time).
    v8 kn[KS], vn[DT][2];
    auto fetch_k = [&](int t) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kn[ks] = ld8<E>(p1_at<E, D>(KP, t, ks, lane));
    };
    auto fetch_v = [&](int t) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
                vn[dt][kk] = ld8<E>(p2_at<E, D>(VP2, t, dt, kk, lane));
    };
    float b[16];  // per-key bias of the tile (0 without one), fetched ahead like the operands
#pragma unroll
    for (int i = 0; i < 16; ++i) b[i] = 0.f;
    auto fetch_b = [&](int t) {
        if (bias) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const float4 v = *reinterpret_cast<const float4*>(bias + t * 32 + 16 * h + 8 * g + 4 * c);
                    b[8 * h + 4 * c] = v.x; b[8 * h + 4 * c + 1] = v.y; b[8 * h + 4 * c + 2] = v.z; b[8 * h + 4 * c + 3] = v.w;
                }
        }
    };
    const int t_first = a_lo / 32 + wave, t_last = a_hi / 32;
    if (t_first <= t_last) {
        fetch_k(t_first);
        fetch_b(t_first);
        fetch_v(t_first);
    }
    for (int t = t_first; t <= t_last; t += kW) {
        const int a0 = t * 32;
        const bool more = t + kW <= t_last;
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = M::mma(kn[ks], xb[ks], s);
        if (more) fetch_k(t + kW);
        // Only tiles on an edge of the band (or past the end of the sequence) need the element-wise mask.
        const bool edge = (a0 + 31 >= T) || (p.causal && ((a0 + 31 > r0) || (r0 + 31 - a0 > p.k_diff)));
        float sv[16];
        if (edge) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int a = a0 + key_of(g, i);
                const bool ok = (a < T) & ((!p.causal) | ((a <= r) & (r - a <= p.k_diff)));
                sv[i] = ok ? fmaf(s[i], p.scale_log2, b[i]) : -INFINITY;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) sv[i] = fmaf(s[i], p.scale_log2, b[i]);
        }
        if (more) fetch_b(t + kW);
        float tmax = fmaxf(sv[0], sv[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) tmax = fmaxf(fmaxf(tmax, sv[i]), sv[i + 1]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        // The reference maximum is raised lazily: only when some row's scores exceed it by more than 2^8
        // (the first tile always does: m starts at -inf), so most tiles skip the rescaling.
        if (__any(tmax > m + kLazyRaise)) {
            const float m_new = fmaxf(m, tmax);
            const float f = fast_exp2(m - (m_new == -INFINITY ? 0.f : m_new));
            m = m_new;
            l *= f;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[dt][i] *= f;
        }
        const float m_use = m == -INFINITY ? 0.f : m;
        v8 pb[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const typename M::v2 pr = M::pack(fast_exp2(sv[8 * h + e] - m_use), fast_exp2(sv[8 * h + e + 1] - m_use));
                l = M::add_pair(pr, l);  // the row sum of what the value product sees
                pb[h][e] = pr[0];
                pb[h][e + 1] = pr[1];
            }
        // O^T[d][r] += V^T[d][a] P^T[a][r]
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
                acc[dt] = M::mma(vn[dt][kk], pb[kk], acc[dt]);
        if (more) fetch_v(t + kW);
    }
    l += __shfl_xor(l, 32, 64);

    // merge the waves' partial softmaxes
    if (g == 0) {
        sM[wave * 32 + n] = m;
        sL[wave * 32 + n] = l;
    }
    spill_tiles<D>(sO, wave, acc, n, g);
    __syncthreads();
    const int rr = tid & 31, dg = tid >> 5, row = r0 + rr;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kW; ++w) mm = fmaxf(mm, sM[w * 32 + rr]);
    float e[kW], ll = 0.f;
#pragma unroll
    for (int w = 0; w < kW; ++w) {
        const float mw = sM[w * 32 + rr];
        e[w] = mw == -INFINITY ? 0.f : fast_exp2(mw - mm);
        ll += e[w] * sL[w * 32 + rr];
    }
    const float inv = 1.0f / ll;
    if (dg == 0 && row < T) p.lse[(size_t)bh * p.lse_stride + row] = (mm + fast_log2(ll)) * p.lse_scale;
#pragma unroll
    for (int c = dg; c < D / 8; c += 2 * kW) {  // 16-byte pieces dg, dg + 2 kW, ... of the row
        const int d0 = 8 * c;
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kW; ++w) v += e[w] * sO[(w * D + d0 + j) * kLdr + rr];
            o[j] = v * inv;
        }
        const size_t off = base + (size_t)row * D + d0;
        if (row < T) {
            if (p.out) {
                v8 ov;
#pragma unroll
                for (int j = 0; j < 8; ++j) ov[j] = (E)o[j];
                *reinterpret_cast<v8*>(p.out + off) = ov;
            }
            if (p.out_f32) {
                *reinterpret_cast<float4*>(p.out_f32 + off) = make_float4(o[0], o[1], o[2], o[3]);
                *reinterpret_cast<float4*>(p.out_f32 + off + 4) = make_float4(o[4], o[5], o[6], o[7]);
            }
        }
        if (p.mul) {
            v8 mv;
#pragma unroll
            for (int j = 0; j < 8; ++j) mv[j] = (E)0.f;
            if (row < T) mv = ld8<E>(p.mul.row(at, row, T, D) + d0);
            v8 wv;
#pragma unroll
            for (int j = 0; j < 8; ++j) wv[j] = (E)(row < T ? o[j] * (float)mv[j] : 0.f);
            if (p.outm && row < T) *reinterpret_cast<v8*>(p.outm + off) = wv;
            if (p.outm_p1) *reinterpret_cast<v8*>(p.outm_p1 + tb + p1_index<D>(row, d0)) = wv;  // 8 consecutive d: one piece
            if (p.outm_p2)
#pragma unroll
                for (int j = 0; j < 8; ++j) p.outm_p2[tb + p2_index<D>(row, d0 + j)] = wv[j];
        }
    }
    }  // owner tiles of this workgroup
}

#include "dps_fwd_shared.hpp"

// ------------------------------------------------------------------------------ backward, rows
template <typename E, bool SV>
struct AttnBwdP {
    // row-major: what the owner tile loads once (row kernel: x, g; column kernel: k, v)
    View<E, SV> x, g, k, v;
    // streamed, operand-packed [BH][Tp*D]: row kernel kp, vp (P1) and kp2 (P2);
    // column kernel xp, gp (P1) and xp2, gp2 (P2)
    const E *kp, *vp, *kp2, *xp, *gp, *xp2, *gp2;
    const float* bias;       // [BH][Tp] log2 units or null
    const float* lse2;       // [BH][Tp] log2 units
    const float* delta;      // [BH][Tp]
    int BH, T, Tp;
    int H;                   // heads per batch entry in the views' indexing
    float alpha;
    int causal, k_diff;
    int pair;                // a workgroup takes two owner tiles, a long and a short one (see owner_tiles)
    // row kernel output: dx = alpha * sum + addend
    const float* addend;     // fp32 [BH][T][D] or null
    E* dx;
    // column kernel outputs
    float* dk_f32;           // alpha * sum  (fp32) or null
    E* dk;                   // alpha * sum  (16 bit) or null
    // LINK == false: dv = sum * SiLU'(v1)
    View<E, SV> v1;
    E* dv;
    // LINK == true: dW = sum;  dV2 = dW R;  dR = dW V2;  delta1 = rowsum(dR R) - dbias
    const float* r_f32;
    View<E, SV> v2;
    E *dv2, *dr, *dr_p1, *dr_p2;
    float* delta1;           // [BH][Tp]
};

template <typename E, int D, int kW, bool SV>
__device__ __forceinline__ void attn_bwd_row_body(const AttnBwdP<E, SV>& p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    constexpr int KS = D / 16, DT = D / 32;
    extern __shared__ __align__(16) char smem_raw[];
    float* sO = reinterpret_cast<float*>(smem_raw);  // [kW][D][kLdr]

    int bh, tile0;
    if (!block_to_tile(p.BH, launch_tiles(p.pair, p.Tp / 32), bh, tile0)) return;
    const int nparts = owner_tiles(p.pair, p.Tp / 32, tile0);
    for (int op = 0; op < nparts; ++op) {
    if (op) __syncthreads();  // the merge tiles of the first owner tile have been read
    const int tile = owner_tile(p.Tp / 32, tile0, op);
    const int r0 = (p.Tp / 32 - 1 - tile) * 32;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T, Tp = p.Tp;
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp, vb = (size_t)bh * Tp;
    const E* __restrict__ KP = p.kp + tb;
    const E* __restrict__ VP = p.vp + tb;
    const E* __restrict__ KP2 = p.kp2 + tb;
    const float* __restrict__ bias = p.bias ? p.bias + vb : nullptr;
    const int r = r0 + n, rc = min(r, T - 1);
    const float scale_log2 = p.alpha * kLog2e;

    const int2 at = slice_at<SV>(bh, p.H);
    v8 xb[KS], gb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        xb[ks] = ld8<E>(p.x.row(at, rc, T, D) + 16 * ks + 8 * g);
        gb[ks] = ld8<E>(p.g.row(at, rc, T, D) + 16 * ks + 8 * g);
    }
    const float lse2 = p.lse2[vb + rc], dl = p.delta[vb + rc];

    const int a_lo = p.causal ? max(0, r0 - p.k_diff) : 0;
    const int a_hi = p.causal ? min(T - 1, r0 + 31) : T - 1;
    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

    // streamed operands and the bias of a tile are fetched one tile ahead, into the registers the
    // previous tile has just consumed
    v8 kn[KS], vn[KS], k2n[DT][2];
    float b[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) b[i] = 0.f;
    auto fetch_rows = [&](int t) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            kn[ks] = ld8<E>(p1_at<E, D>(KP, t, ks, lane));
            vn[ks] = ld8<E>(p1_at<E, D>(VP, t, ks, lane));
        }
    };
    auto fetch_bias = [&](int t) {
        if (bias) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const float4 v = *reinterpret_cast<const float4*>(bias + t * 32 + 16 * h + 8 * g + 4 * c);
                    b[8 * h + 4 * c] = v.x; b[8 * h + 4 * c + 1] = v.y; b[8 * h + 4 * c + 2] = v.z; b[8 * h + 4 * c + 3] = v.w;
                }
        }
    };
    auto fetch_cols = [&](int t) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) k2n[dt][kk] = ld8<E>(p2_at<E, D>(KP2, t, dt, kk, lane));
    };
    const int t_first = a_lo / 32 + wave, t_last = a_hi / 32;
    if (t_first <= t_last) {
        fetch_rows(t_first);
        fetch_bias(t_first);
        fetch_cols(t_first);
    }
    for (int t = t_first; t <= t_last; t += kW) {
        const int a0 = t * 32;
        const bool more = t + kW <= t_last;
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = 0.f;
            dp[i] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = M::mma(kn[ks], xb[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = M::mma(vn[ks], gb[ks], dp);
        if (more) fetch_rows(t + kW);
        // only tiles on an edge of the band (or past the end of the sequence) need the element-wise mask
        const bool edge = (a0 + 31 >= T) || (r0 + 31 >= T) || (p.causal && ((a0 + 31 > r0) || (r0 + 31 - a0 > p.k_diff)));
        float ds[16];
        if (edge) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int a = a0 + key_of(g, i);
                const bool ok = pair_ok(T, p.causal, p.k_diff, r, a);
                const float pr = ok ? fast_exp2(fmaf(s[i], scale_log2, b[i] - lse2)) : 0.f;
                ds[i] = pr * (dp[i] - dl);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) ds[i] = fast_exp2(fmaf(s[i], scale_log2, b[i] - lse2)) * (dp[i] - dl);
        }
        if (more) fetch_bias(t + kW);
        v8 dsb[2];
        pack16<E>(ds, dsb);
        // dX^T[d][r] += K^T[d][a] dS^T[a][r]
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) acc[dt] = M::mma(k2n[dt][kk], dsb[kk], acc[dt]);
        if (more) fetch_cols(t + kW);
    }

    spill_tiles<D>(sO, wave, acc, n, g);
    __syncthreads();
    const int rr = tid & 31, dg = tid >> 5, row = r0 + rr;
#pragma unroll
    for (int c = dg; c < D / 8; c += 2 * kW) {  // 16-byte pieces dg, dg + 2 kW, ... of the row
        if (row >= T) break;
        const int d0 = 8 * c;
        const size_t off = base + (size_t)row * D + d0;
        v8 ov;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kW; ++w) v += sO[(w * D + d0 + j) * kLdr + rr];
            v *= p.alpha;
            if (p.addend) v += p.addend[off + j];
            ov[j] = (E)v;
        }
        *reinterpret_cast<v8*>(p.dx + off) = ov;
    }
    }  // owner tiles of this workgroup
}

template <typename E, int D, int kW, bool SV>
__global__ __launch_bounds__(64 * kW, (D <= 64 ? 2 : 1)) void attn_bwd_row_mfma_kernel(AttnBwdP<E, SV> p) {
    attn_bwd_row_body<E, D, kW, SV>(p);
}
// Two row passes in one grid (blockIdx.y picks the pass): the outer pass's dQ and the inner pass's dK2 depend on
// nothing of each other, and one pass alone gives a SIMD a single latency-bound wave.
template <typename E, int D, int kW, bool SV>
__global__ __launch_bounds__(64 * kW, (D <= 64 ? 2 : 1)) void attn_bwd_row_pair_kernel(AttnBwdP<E, SV> p0, AttnBwdP<E, SV> p1) {
    attn_bwd_row_body<E, D, kW, SV>(blockIdx.y == 0 ? p0 : p1);
}

// --------------------------------------------------------------------------- backward, columns
// RING: every wave fetches its streamed tiles into a two-slot LDS ring of its own (direct-to-LDS loads, one tile ahead)
// and reads the MFMA operands and the rows' statistics from there at the point of use, instead of holding the next
// tile in registers: the kernel then fits 256 registers and two waves per SIMD (D = 64: 36 KB of LDS per wave).
template <int D>
constexpr int col_ring_tile_bytes() { return 4 * (D / 16) * 1024 + 2 * 256; }
template <typename E, int D, int kW, bool LINK, bool SV, bool RING = false>
__global__ __launch_bounds__(64 * kW, ((D <= 32 || RING) ? 2 : 1)) void attn_bwd_col_mfma_kernel(AttnBwdP<E, SV> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    constexpr int KS = D / 16, DT = D / 32;
    constexpr int kTileBytes = col_ring_tile_bytes<D>();
    extern __shared__ __align__(16) char smem_raw[];
    float* sO = reinterpret_cast<float*>(smem_raw);  // [kW][D][kLdr]
    float* sB = sO + kW * D * kLdr;                  // [kW][32]  dbias partials
    float* sR = sB + kW * 32;                        // [2 kW][32]   delta1 partials

    int bh, tile0;
    if (!block_to_tile(p.BH, launch_tiles(p.pair, p.Tp / 32), bh, tile0)) return;
    const int nparts = owner_tiles(p.pair, p.Tp / 32, tile0);
    for (int op = 0; op < nparts; ++op) {
    if (op) __syncthreads();  // the merge tiles of the first owner tile have been read
    const int tile = owner_tile(p.Tp / 32, tile0, op);
    const int c0 = tile * 32;  // lowest key rows are the longest
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T, Tp = p.Tp;
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp, vb = (size_t)bh * Tp;
    const E* __restrict__ XP = p.xp + tb;
    const E* __restrict__ GP = p.gp + tb;
    const E* __restrict__ XP2 = p.xp2 + tb;
    const E* __restrict__ GP2 = p.gp2 + tb;
    const float* __restrict__ lse2 = p.lse2 + vb;
    const float* __restrict__ delta = p.delta + vb;
    const int a = c0 + n, ac = min(a, T - 1);
    const float scale_log2 = p.alpha * kLog2e;

    const int2 at = slice_at<SV>(bh, p.H);
    v8 kb[KS], vbv[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kb[ks] = ld8<E>(p.k.row(at, ac, T, D) + 16 * ks + 8 * g);
        vbv[ks] = ld8<E>(p.v.row(at, ac, T, D) + 16 * ks + 8 * g);
    }
    const float ba = p.bias ? p.bias[vb + ac] : 0.f;

    const int r_lo = p.causal ? c0 : 0;
    const int r_hi = p.causal ? (int)min((long)T - 1, (long)c0 + 31 + p.k_diff) : T - 1;
    f32x16 acck[DT], accv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acck[dt][i] = 0.f;
            accv[dt][i] = 0.f;
        }
    float db = 0.f;

    const int t_first = r_lo / 32 + wave, t_last = r_hi / 32;
    if constexpr (RING) {
        char* ring = smem_raw + wave * 2 * kTileBytes;  // the merge tiles alias the rings: barrier before they are written
        const char* XPc = reinterpret_cast<const char*>(uniform_ptr(XP));
        const char* GPc = reinterpret_cast<const char*>(uniform_ptr(GP));
        const char* XP2c = reinterpret_cast<const char*>(uniform_ptr(XP2));
        const char* GP2c = reinterpret_cast<const char*>(uniform_ptr(GP2));
        auto fetch = [&](int t, int slot) {
            char* dst = ring + __builtin_amdgcn_readfirstlane(slot * kTileBytes);
            const size_t tile_off = (size_t)__builtin_amdgcn_readfirstlane(t) * KS * 1024;
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                direct_load_16(uniform_ptr(XPc + tile_off + c * 1024), lane * 16, dst + c * 1024);
                direct_load_16(uniform_ptr(GPc + tile_off + c * 1024), lane * 16, dst + (KS + c) * 1024);
                direct_load_16(uniform_ptr(XP2c + tile_off + c * 1024), lane * 16, dst + (2 * KS + c) * 1024);
                direct_load_16(uniform_ptr(GP2c + tile_off + c * 1024), lane * 16, dst + (3 * KS + c) * 1024);
            }
            const unsigned voff = (unsigned)min(t * 32 + lane, Tp - 1) * 4;
            direct_load_4(lse2, voff, dst + 4 * KS * 1024);
            direct_load_4(delta, voff, dst + 4 * KS * 1024 + 256);
        };
        if (t_first <= t_last) fetch(t_first, 0);
        int slot = 0;
        for (int t = t_first; t <= t_last; t += kW) {
            const int r0 = t * 32;
            // tile t has landed, and this wave's reads of the other slot are done: it may be overwritten
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));
            asm volatile("" ::: "memory");
            if (t + kW <= t_last) fetch(t + kW, slot ^ 1);
            const char* st = ring + slot * kTileBytes;
            slot ^= 1;
            f32x16 s, dp;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                s[i] = 0.f;
                dp[i] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = M::mma(*reinterpret_cast<const v8*>(st + ks * 1024 + lane * 16), kb[ks], s);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) dp = M::mma(*reinterpret_cast<const v8*>(st + (KS + ks) * 1024 + lane * 16), vbv[ks], dp);
            float ls[16], dl[16];
            tile_vector(reinterpret_cast<const float*>(st + 4 * KS * 1024), g, ls);
            tile_vector(reinterpret_cast<const float*>(st + 4 * KS * 1024 + 256), g, dl);
            const bool edge = (r0 + 31 >= T) || (c0 + 31 >= T) || (p.causal && ((c0 + 31 > r0) || (r0 + 31 - c0 > p.k_diff)));
            float pr[16], ds[16];
            if (edge) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int r = r0 + key_of(g, i);
                    const bool ok = pair_ok(T, p.causal, p.k_diff, r, a);
                    pr[i] = ok ? fast_exp2(fmaf(s[i], scale_log2, ba - ls[i])) : 0.f;
                    ds[i] = ok ? pr[i] * (dp[i] - dl[i]) : 0.f;
                    db += ds[i];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    pr[i] = fast_exp2(fmaf(s[i], scale_log2, ba - ls[i]));
                    ds[i] = pr[i] * (dp[i] - dl[i]);
                    db += ds[i];
                }
            }
            v8 pb[2], dsb[2];
            pack16<E>(pr, pb);
            pack16<E>(ds, dsb);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
                    acck[dt] = M::mma(*reinterpret_cast<const v8*>(st + (2 * KS + dt * 2 + kk) * 1024 + lane * 16), dsb[kk], acck[dt]);
                    accv[dt] = M::mma(*reinterpret_cast<const v8*>(st + (3 * KS + dt * 2 + kk) * 1024 + lane * 16), pb[kk], accv[dt]);
                }
        }
        __syncthreads();  // every wave is done with its ring: the merge tiles go on top of them
    } else {
    // streamed operands and the per-row statistics of a tile are fetched one tile ahead, into the
    // registers the previous tile has just consumed
    v8 xn[KS], gn[KS], x2n[DT][2], g2n[DT][2];
    float ls[16], dl[16];
    auto fetch_rows = [&](int t) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            xn[ks] = ld8<E>(p1_at<E, D>(XP, t, ks, lane));
            gn[ks] = ld8<E>(p1_at<E, D>(GP, t, ks, lane));
        }
    };
    auto fetch_stats = [&](int t) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const float4 v = *reinterpret_cast<const float4*>(lse2 + t * 32 + 16 * h + 8 * g + 4 * c);
                const float4 w = *reinterpret_cast<const float4*>(delta + t * 32 + 16 * h + 8 * g + 4 * c);
                ls[8 * h + 4 * c] = v.x; ls[8 * h + 4 * c + 1] = v.y; ls[8 * h + 4 * c + 2] = v.z; ls[8 * h + 4 * c + 3] = v.w;
                dl[8 * h + 4 * c] = w.x; dl[8 * h + 4 * c + 1] = w.y; dl[8 * h + 4 * c + 2] = w.z; dl[8 * h + 4 * c + 3] = w.w;
            }
    };
    auto fetch_cols = [&](int t) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                x2n[dt][kk] = ld8<E>(p2_at<E, D>(XP2, t, dt, kk, lane));
                g2n[dt][kk] = ld8<E>(p2_at<E, D>(GP2, t, dt, kk, lane));
            }
    };
    if (t_first <= t_last) {
        fetch_rows(t_first);
        fetch_stats(t_first);
        fetch_cols(t_first);
    }
    for (int t = t_first; t <= t_last; t += kW) {
        const int r0 = t * 32;
        const bool more = t + kW <= t_last;
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = 0.f;
            dp[i] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = M::mma(xn[ks], kb[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = M::mma(gn[ks], vbv[ks], dp);
        if (more) fetch_rows(t + kW);
        // only tiles on an edge of the band (or past the end of the sequence) need the element-wise mask
        const bool edge = (r0 + 31 >= T) || (c0 + 31 >= T) || (p.causal && ((c0 + 31 > r0) || (r0 + 31 - c0 > p.k_diff)));
        float pr[16], ds[16];
        if (edge) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int r = r0 + key_of(g, i);
                const bool ok = pair_ok(T, p.causal, p.k_diff, r, a);
                pr[i] = ok ? fast_exp2(fmaf(s[i], scale_log2, ba - ls[i])) : 0.f;
                ds[i] = ok ? pr[i] * (dp[i] - dl[i]) : 0.f;
                db += ds[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                pr[i] = fast_exp2(fmaf(s[i], scale_log2, ba - ls[i]));
                ds[i] = pr[i] * (dp[i] - dl[i]);
                db += ds[i];
            }
        }
        if (more) fetch_stats(t + kW);
        v8 pb[2], dsb[2];
        pack16<E>(pr, pb);
        pack16<E>(ds, dsb);
        // dK^T[d][a] += X^T[d][r] dS[r][a];  dV^T[d][a] += G^T[d][r] P[r][a]
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                acck[dt] = M::mma(x2n[dt][kk], dsb[kk], acck[dt]);
                accv[dt] = M::mma(g2n[dt][kk], pb[kk], accv[dt]);
            }
        if (more) fetch_cols(t + kW);
    }
    }  // operands from registers
    db += __shfl_xor(db, 32, 64);

    const int aa = tid & 31, dg = tid >> 5, row = c0 + aa;
    // ---- dK
    if (g == 0) sB[wave * 32 + n] = db;
    spill_tiles<D>(sO, wave, acck, n, g);
    __syncthreads();
    if (row < T) {
#pragma unroll
        for (int c = dg; c < D / 8; c += 2 * kW) {
            const int d0 = 8 * c;
            const size_t off = base + (size_t)row * D + d0;
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float v = 0.f;
#pragma unroll
                for (int w = 0; w < kW; ++w) v += sO[(w * D + d0 + j) * kLdr + aa];
                o[j] = v * p.alpha;
            }
            if (p.dk_f32) {
                *reinterpret_cast<float4*>(p.dk_f32 + off) = make_float4(o[0], o[1], o[2], o[3]);
                *reinterpret_cast<float4*>(p.dk_f32 + off + 4) = make_float4(o[4], o[5], o[6], o[7]);
            }
            if (p.dk) {
                v8 ov;
#pragma unroll
                for (int j = 0; j < 8; ++j) ov[j] = (E)o[j];
                *reinterpret_cast<v8*>(p.dk + off) = ov;
            }
        }
    }
    __syncthreads();
    // ---- dV
    spill_tiles<D>(sO, wave, accv, n, g);
    __syncthreads();
    float part = 0.f;
#pragma unroll
    for (int c = dg; c < D / 8; c += 2 * kW) {  // 16-byte pieces dg, dg + 2 kW, ... of the row
        const int d0 = 8 * c;
        const size_t off = base + (size_t)row * D + d0;
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < kW; ++w) v += sO[(w * D + d0 + j) * kLdr + aa];
            o[j] = v;
        }
        if constexpr (!LINK) {
            if (row < T) {
                const v8 x = ld8<E>(p.v1.row(at, row, T, D) + d0);
                v8 ov;
#pragma unroll
                for (int j = 0; j < 8; ++j) ov[j] = (E)(o[j] * silu_grad_f((float)x[j]));
                *reinterpret_cast<v8*>(p.dv + off) = ov;
            }
        } else {
            v8 dv2, dr;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                dv2[j] = (E)0.f;
                dr[j] = (E)0.f;
            }
            if (row < T) {
                const v8 x = ld8<E>(p.v2.row(at, row, T, D) + d0);
                const float4 ra = *reinterpret_cast<const float4*>(p.r_f32 + off);
                const float4 rb = *reinterpret_cast<const float4*>(p.r_f32 + off + 4);
                const float rv[8] = {ra.x, ra.y, ra.z, ra.w, rb.x, rb.y, rb.z, rb.w};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float drj = o[j] * (float)x[j];
                    dv2[j] = (E)(o[j] * rv[j]);
                    dr[j] = (E)drj;
                    part += drj * rv[j];
                }
                *reinterpret_cast<v8*>(p.dv2 + off) = dv2;
                *reinterpret_cast<v8*>(p.dr + off) = dr;
            }
            *reinterpret_cast<v8*>(p.dr_p1 + tb + p1_index<D>(row, d0)) = dr;  // zeros for the padding rows
#pragma unroll
            for (int j = 0; j < 8; ++j) p.dr_p2[tb + p2_index<D>(row, d0 + j)] = dr[j];
        }
    }
    if constexpr (LINK) {
        sR[dg * 32 + aa] = part;
        __syncthreads();
        if (tid < 32) {
            float d1 = 0.f;
#pragma unroll
            for (int j = 0; j < 2 * kW; ++j) d1 += sR[j * 32 + tid];
#pragma unroll
            for (int w = 0; w < kW; ++w) d1 -= sB[w * 32 + tid];
            p.delta1[vb + c0 + tid] = (c0 + tid < T) ? d1 : 0.f;
        }
    }
    }  // owner tiles of this workgroup
}

#include "dps_bwd_shared.hpp"

// --------------------------------------------------------------------------------------- prep
// Operand-packed copies of the inputs (U = SiLU(V1); rows past T are written as zeros), U row-major, and
// the padded per-row vectors of the backward (LSE in log2 units, Delta = rowsum(dO * O)).  Null
// pointers are skipped.
template <typename E, bool SV>
struct PrepP {
    View<E, SV> v1, k1, k2, q, d_o;
    const E* o;  // dense: the library's own output
    const float* lse;
    E* u;                            // row-major
    E *up1, *k1p1, *k2p1, *qp1, *dop1;  // packing P1
    E *up2, *k1p2, *k2p2, *qp2, *dop2;  // packing P2
    float *lse2, *delta;
    int BH, T, Tp;
    int H;  // heads per batch entry in the views' indexing
};

template <typename E, int D, bool SV>
__global__ __launch_bounds__(256) void dps_prep_kernel(PrepP<E, SV> p) {
    using v8 = typename Mma<E>::v8;
    int bh, tile_id;
    if (!block_to_tile(p.BH, p.Tp / 32, bh, tile_id)) return;
    const int j0 = tile_id * 32, T = p.T, Tp = p.Tp;
    const int2 at = slice_at<SV>(bh, p.H);
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp;
    // One 16-byte piece (8 consecutive d of one row) per thread and step: it is one piece of P1 as it stands.
    // P2 wants 8 consecutive rows of one column in a piece, so the 32 x D tile goes through LDS and comes
    // back out transposed, again as whole 16-byte pieces (element-wise 2-byte stores were most of this
    // kernel's time).
    __shared__ E sT[32][D + 2];
    auto emit = [&](const View<E, SV>& src, E* dst1, E* dst2, bool silu) {
        if (!dst1 && !dst2 && !(silu && p.u)) return;  // uniform over the workgroup
        for (int idx = threadIdx.x; idx < 32 * (D / 8); idx += 256) {
            const int jj = idx / (D / 8), j = j0 + jj, d0 = (idx % (D / 8)) * 8;
            const bool in = j < T;
            const size_t off = base + (size_t)(in ? j : 0) * D + d0;
            v8 x;
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (E)0.f;
            if (in) x = *reinterpret_cast<const v8*>(src.row(at, j, T, D) + d0);
            if (silu) {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (E)(in ? silu_f((float)x[e]) : 0.f);
                if (p.u && in) *reinterpret_cast<v8*>(p.u + off) = x;
            }
            if (dst1) *reinterpret_cast<v8*>(dst1 + tb + p1_index<D>(j, d0)) = x;
            if (dst2) {
#pragma unroll
                for (int e = 0; e < 8; ++e) sT[jj][d0 + e] = x[e];
            }
        }
        if (dst2) {
            __syncthreads();
            for (int idx = threadIdx.x; idx < (D / 32) * 2 * 64; idx += 256) {
                const int ln = idx & 63, kk = (idx >> 6) & 1, dt = idx >> 7;
                const int r = kk * 16 + (ln >> 5) * 8, d = dt * 32 + (ln & 31);
                v8 y;
#pragma unroll
                for (int e = 0; e < 8; ++e) y[e] = sT[r + e][d];
                *reinterpret_cast<v8*>(dst2 + tb + ((size_t)((tile_id * (D / 32) + dt) * 2 + kk) * 64 + ln) * 8) = y;
            }
            __syncthreads();
        }
    };
    // blockIdx.y deals the tensors out (3 in the forward, 5 and the row vectors in the backward): a workgroup per
    // tile walking them one after the other was five dependent round trips through LDS
    const int job = blockIdx.y;
    if (job == 0) emit(p.v1, p.up1, p.up2, true);
    if (job == 1) emit(p.k1, p.k1p1, p.k1p2, false);
    if (job == 2) emit(p.k2, p.k2p1, p.k2p2, false);
    if (job == 3 && p.q) emit(p.q, p.qp1, p.qp2, false);
    if (job == 4 && p.d_o) emit(p.d_o, p.dop1, p.dop2, false);
    if (job == 5 && p.delta) {
        // Delta[j] = dO[j] . O[j]: the D / 8 lanes that hold a row's 16-byte pieces sit next to each other
        constexpr int cpr = D / 8;
        for (int idx = threadIdx.x; idx < 32 * cpr; idx += 256) {
            const int j = j0 + idx / cpr, c = idx % cpr;
            float part = 0.f;
            if (j < T) {
                const size_t off = base + (size_t)j * D + c * 8;
                const v8 a = *reinterpret_cast<const v8*>(p.o + off), b = *reinterpret_cast<const v8*>(p.d_o.row(at, j, T, D) + c * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e) part += (float)a[e] * (float)b[e];
            }
#pragma unroll
            for (int off = cpr >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
            if (c == 0) {
                p.delta[(size_t)bh * Tp + j] = part;
                p.lse2[(size_t)bh * Tp + j] = j < T ? p.lse[(size_t)bh * T + j] * kLog2e : 0.f;
            }
        }
    }
}

struct Layout {
    size_t up2, k1p1, k2p1, wp2, lse1;                                            // forward
    size_t u, up1, k1p2, k2p2, qp1, qp2, dop1, dop2, w, wp1, dr, drp1, drp2, r, dk2p, lse2, delta, delta1;  // backward
    size_t total;
};
Layout layout(int BH, int T, int D, bool bwd) {
    const size_t Tp = (size_t)(T + 31) / 32 * 32, n = (size_t)BH * T * D, nt = (size_t)BH * D * Tp, nv = (size_t)BH * Tp;
    Layout l{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        off = (off + 255) & ~size_t(255);
        const size_t r = off;
        off += bytes;
        return r;
    };
    l.up2 = take(nt * 2);
    l.k1p1 = take(nt * 2);
    l.k2p1 = take(nt * 2);
    l.wp2 = take(nt * 2);
    l.lse1 = take(nv * 4);
    if (bwd) {
        l.u = take(n * 2);
        l.up1 = take(nt * 2);
        l.k1p2 = take(nt * 2);
        l.k2p2 = take(nt * 2);
        l.qp1 = take(nt * 2);
        l.qp2 = take(nt * 2);
        l.dop1 = take(nt * 2);
        l.dop2 = take(nt * 2);
        l.w = take(n * 2);
        l.wp1 = take(nt * 2);
        l.dr = take(n * 2);
        l.drp1 = take(nt * 2);
        l.drp2 = take(nt * 2);
        l.r = take(n * 4);
        l.dk2p = take(n * 4);
        l.lse2 = take(nv * 4);
        l.delta = take(nv * 4);
        l.delta1 = take(nv * 4);
    }
    l.total = (off + 255) & ~size_t(255);
    return l;
}

template <int D, int kW>
constexpr size_t fwd_smem() { return 4 * (size_t)(kW * D * kLdr + 2 * kW * 32); }
template <int D, int kW, bool RING = false>
constexpr size_t col_smem() {
    const size_t merge = 4 * (size_t)(kW * D * kLdr + kW * 32 + 2 * kW * 32), ring = (size_t)kW * 2 * col_ring_tile_bytes<D>();
    return RING && ring > merge ? ring : merge;
}
template <int D, int kW>
constexpr size_t row_smem() { return 4 * (size_t)(kW * D * kLdr); }

template <typename F>
hipError_t allow_smem(F kern, size_t bytes) {
    return ensure_dynamic_smem(reinterpret_cast<const void*>(kern), bytes);
}
// Owner tiles are paired (owner_tiles) when the pass is a full causal triangle of at least 32 tiles and the halved
// grid still gives every CU two workgroups; measured together with the wave count (dps_waves below).
bool pair_tiles(const MfmaDpsArgs& a, int k_diff, int workgroups, bool backward) {
    const int knob = knobs().dps_pair;
    if (knob) return knob > 0;
    return a.causal && k_diff >= a.T - 1 && workgroups >= 1024 && a.T >= (backward ? 2048 : 1024);
}
dim3 attn_grid(const MfmaDpsArgs& a, int Tp, bool pair) {
    const int nt = Tp / 32;
    return dim3(8 * xcd_slots(a.BH, pair ? (nt + 1) / 2 : nt));
}

// one of the caller's tensors / a row-major tensor of the workspace as the kernels take them
// one of the caller's tensors / a row-major tensor of the workspace as the kernels take them
template <typename E, bool SV>
View<E, SV> dense_view(const MfmaDpsArgs& a, const void* p) {
    if constexpr (SV) return View<E, true>{(const E*)p, (long long)a.H * a.T * a.D, (long long)a.T * a.D, (unsigned)a.D};
    else return View<E, false>{(const E*)p};
}
template <typename E, bool SV>
View<E, SV> caller_view(const MfmaDpsArgs& a, const void* p, const RowLayout& l) {
    if constexpr (SV) return View<E, true>{(const E*)p, l.sb, l.sh, (unsigned)l.st};
    else return View<E, false>{(const E*)p};
}

template <typename E, int D, int kW, bool SV>
hipError_t run_fwd(const MfmaDpsArgs& a, hipStream_t st, bool for_bwd) {
    const int Tp = (a.T + 31) / 32 * 32;
    const Layout l = layout(a.BH, a.T, D, for_bwd);
    char* ws = static_cast<char*>(a.workspace);
    const dim3 grid(8 * xcd_slots(a.BH, Tp / 32));
    const bool pair_in = pair_tiles(a, a.k_diff, grid.x, for_bwd), pair_out = pair_tiles(a, a.T, grid.x, for_bwd);
    auto kern = attn_fwd_mfma_kernel<E, D, kW, SV>;
    hipError_t e = allow_smem(kern, fwd_smem<D, kW>());
    if (e != hipSuccess) return e;
    const float sl2 = a.alpha * kLog2e;

    if (!for_bwd) {  // the backward's prep kernel has already written these
        PrepP<E, SV> pp{};
        pp.v1 = caller_view<E, SV>(a, a.v1, a.lv1); pp.k1 = caller_view<E, SV>(a, a.k1, a.lk1); pp.k2 = caller_view<E, SV>(a, a.k2, a.lk2);
        pp.up2 = (E*)(ws + l.up2); pp.k1p1 = (E*)(ws + l.k1p1); pp.k2p1 = (E*)(ws + l.k2p1);
        pp.BH = a.BH; pp.T = a.T; pp.Tp = Tp; pp.H = a.H;
        hipLaunchKernelGGL((dps_prep_kernel<E, D, SV>), dim3(grid.x, 3), dim3(256), 0, st, pp);
    }
    // inner: rows K2[t], keys K1, values U; R (fp32, backward only), W = R * V2 and W^T, lse1 (log2)
    AttnFwdP<E, SV> p{};
    p.x = caller_view<E, SV>(a, a.k2, a.lk2); p.kp = (const E*)(ws + l.k1p1); p.vp2 = (const E*)(ws + l.up2);
    p.mul = caller_view<E, SV>(a, a.v2, a.lv2);
    p.out_f32 = for_bwd ? (float*)(ws + l.r) : nullptr;
    p.outm = for_bwd ? (E*)(ws + l.w) : nullptr;
    p.outm_p1 = for_bwd ? (E*)(ws + l.wp1) : nullptr;
    p.outm_p2 = (E*)(ws + l.wp2);
    p.lse = (float*)(ws + l.lse1); p.lse_stride = Tp; p.lse_scale = 1.0f;
    p.BH = a.BH; p.H = a.H; p.T = a.T; p.Tp = Tp; p.scale_log2 = sl2; p.causal = a.causal; p.k_diff = a.k_diff;
    p.pair = pair_in;
    // Large grids take the kernel whose workgroups own 128 rows and share the streamed tiles through LDS
    // (dps_fwd_shared.hpp).  One wave per 32 rows walks all streamed tiles of its rows, so the kernel needs four of
    // its workgroups per CU to keep the SIMDs busy; measured forward, bf16 D = 64, one owner tile per workgroup ->
    // shared tiles: B=8 H=16 T=2048 398 -> 282 us, B=4 H=8 T=4096 305 -> 262 us, but B=1 H=8 T=8192 (512 workgroups)
    // 277 -> 391 us and B=4 H=8 T=1024 (256) 45 -> 70 us.
    constexpr int kSW = 4, kNS = 4;  // its waves and ring slots
    using Shared = FwdSharedShape<D, kSW, kNS>;
    auto kern_in = attn_fwd_shared_kernel<E, D, kSW, kNS, false, SV>;
    auto kern_out = attn_fwd_shared_kernel<E, D, kSW, kNS, true, SV>;
    const int owners = (Tp / 32 + kSW - 1) / kSW;
    const bool shared = knobs().dps_shared ? knobs().dps_shared > 0 : (long long)a.BH * owners >= 1024;
    const dim3 grid_shared(8 * xcd_slots(a.BH, owners));
    if (shared) {
        if (e = allow_smem(kern_in, Shared::smem); e != hipSuccess) return e;
        if (e = allow_smem(kern_out, Shared::smem); e != hipSuccess) return e;
        hipLaunchKernelGGL(kern_in, grid_shared, dim3(64 * kSW), Shared::smem, st, p);
    } else {
        hipLaunchKernelGGL(kern, attn_grid(a, Tp, pair_in), dim3(64 * kW), (fwd_smem<D, kW>()), st, p);
    }
    if (for_bwd) return hipGetLastError();
    // outer: rows Q[q], keys K2 with bias lse1, values W; O and LSE (natural log)
    AttnFwdP<E, SV> o{};
    o.x = caller_view<E, SV>(a, a.q, a.lq); o.kp = (const E*)(ws + l.k2p1); o.vp2 = (const E*)(ws + l.wp2); o.bias = (const float*)(ws + l.lse1);
    o.out = (E*)a.o_out; o.lse = a.lse_out; o.lse_stride = a.T; o.lse_scale = kLn2;
    o.BH = a.BH; o.H = a.H; o.T = a.T; o.Tp = Tp; o.scale_log2 = sl2; o.causal = a.causal; o.k_diff = a.T;
    o.pair = pair_out;
    if (shared) hipLaunchKernelGGL(kern_out, grid_shared, dim3(64 * kSW), Shared::smem, st, o);
    else hipLaunchKernelGGL(kern, attn_grid(a, Tp, pair_out), dim3(64 * kW), (fwd_smem<D, kW>()), st, o);
    return hipGetLastError();
}

template <typename E, int D, int kW, bool SV>
hipError_t run_bwd(const MfmaDpsArgs& a, hipStream_t st) {
    const int Tp = (a.T + 31) / 32 * 32;
    const Layout l = layout(a.BH, a.T, D, true);
    char* ws = static_cast<char*>(a.workspace);
    const dim3 grid(8 * xcd_slots(a.BH, Tp / 32));
    const bool pair_in = pair_tiles(a, a.k_diff, grid.x, true), pair_out = pair_tiles(a, a.T, grid.x, true);
    auto krow = attn_bwd_row_mfma_kernel<E, D, kW, SV>;
    // the column kernel's operands through per-wave LDS rings (see the kernel) where four waves split the streamed tiles,
    // i.e. from T = 2048 on; measured backward, bf16: B=1 H=8 T=4096 306 -> 291 us, B=2 H=8 T=2048 199 -> 191 us; with two
    // waves (B=4 H=8 T=1024) 136.5 -> 138.7 us, so those keep the operands in registers
    constexpr bool kRing = D == 64 && kW == 4;
    auto kcol_link = attn_bwd_col_mfma_kernel<E, D, kW, true, SV, kRing>;
    auto kcol = attn_bwd_col_mfma_kernel<E, D, kW, false, SV, kRing>;
    hipError_t e = allow_smem(krow, row_smem<D, kW>());
    if (e == hipSuccess) e = allow_smem(kcol_link, col_smem<D, kW, kRing>());
    if (e == hipSuccess) e = allow_smem(kcol, col_smem<D, kW, kRing>());
    if (e != hipSuccess) return e;

    PrepP<E, SV> pp{};
    pp.v1 = caller_view<E, SV>(a, a.v1, a.lv1); pp.k1 = caller_view<E, SV>(a, a.k1, a.lk1); pp.k2 = caller_view<E, SV>(a, a.k2, a.lk2);
    pp.q = caller_view<E, SV>(a, a.q, a.lq); pp.d_o = caller_view<E, SV>(a, a.d_o, a.ldo);
    pp.o = (const E*)a.o; pp.lse = a.lse_in;
    pp.u = (E*)(ws + l.u);
    pp.up1 = (E*)(ws + l.up1); pp.k1p1 = (E*)(ws + l.k1p1); pp.k2p1 = (E*)(ws + l.k2p1);
    pp.qp1 = (E*)(ws + l.qp1); pp.dop1 = (E*)(ws + l.dop1);
    pp.up2 = (E*)(ws + l.up2); pp.k1p2 = (E*)(ws + l.k1p2); pp.k2p2 = (E*)(ws + l.k2p2);
    pp.qp2 = (E*)(ws + l.qp2); pp.dop2 = (E*)(ws + l.dop2);
    pp.lse2 = (float*)(ws + l.lse2); pp.delta = (float*)(ws + l.delta);
    pp.BH = a.BH; pp.T = a.T; pp.Tp = Tp; pp.H = a.H;
    hipLaunchKernelGGL((dps_prep_kernel<E, D, SV>), dim3(grid.x, 6), dim3(256), 0, st, pp);
    // recompute the inner pass: R, W, W^T, lse1
    e = run_fwd<E, D, kW, SV>(a, st, true);
    if (e != hipSuccess) return e;

    // outer pass: X = Q, G = dO, K = K2 (bias lse1), V = W
    AttnBwdP<E, SV> o{};
    o.x = caller_view<E, SV>(a, a.q, a.lq); o.g = caller_view<E, SV>(a, a.d_o, a.ldo); o.k = caller_view<E, SV>(a, a.k2, a.lk2);
    o.v = dense_view<E, SV>(a, ws + l.w);
    o.kp = (const E*)(ws + l.k2p1); o.vp = (const E*)(ws + l.wp1); o.kp2 = (const E*)(ws + l.k2p2);
    o.xp = (const E*)(ws + l.qp1); o.gp = (const E*)(ws + l.dop1);
    o.xp2 = (const E*)(ws + l.qp2); o.gp2 = (const E*)(ws + l.dop2);
    o.bias = (const float*)(ws + l.lse1); o.lse2 = (const float*)(ws + l.lse2); o.delta = (const float*)(ws + l.delta);
    o.BH = a.BH; o.H = a.H; o.T = a.T; o.Tp = Tp; o.alpha = a.alpha; o.causal = a.causal; o.k_diff = a.T;
    o.pair = pair_out;
    o.dx = (E*)a.dq;
    o.dk_f32 = (float*)(ws + l.dk2p);
    o.r_f32 = (const float*)(ws + l.r); o.v2 = caller_view<E, SV>(a, a.v2, a.lv2); o.dv2 = (E*)a.dv2;
    o.dr = (E*)(ws + l.dr); o.dr_p1 = (E*)(ws + l.drp1); o.dr_p2 = (E*)(ws + l.drp2); o.delta1 = (float*)(ws + l.delta1);
    // Large grids: the kernels whose workgroups own 128 rows and share the streamed tiles through LDS
    // (dps_bwd_shared.hpp), as the forward passes do (run_fwd).  They pay from 512 such workgroups on; measured
    // backward, bf16 D = 64, one owner tile per workgroup -> shared tiles: B=8 H=16 T=2048 1650 -> 972 us, B=4 H=8
    // T=4096 1245 -> 825 us, B=8 H=16 T=1024 510 -> 376 us, B=4 H=8 T=2048 (512 workgroups) 387 -> 313 us, B=1 H=8
    // T=8192 (512) 1040 -> 1000 us, but B=1 H=8 T=4096 (256) 306 -> 506 us and B=4 H=8 T=1024 (256) 136 -> 175 us;
    // D = 128, B=4 H=8 T=4096: 2120 -> 1935 us.
    constexpr int kSW = 4, kRowNS = 4, kColNS = D > 64 ? 3 : 4;
    using RowShape = BwdSharedShape<D, kSW, kRowNS, 3>;
    using ColShape = BwdSharedShape<D, kSW, kColNS, 4>;
    const int owners = (Tp / 32 + kSW - 1) / kSW;
    bool shared = false;
    if constexpr (D >= 64) shared = knobs().dps_shared ? knobs().dps_shared > 0 : (long long)a.BH * owners >= 512;
    const dim3 grid_shared(8 * xcd_slots(a.BH, owners));
    if constexpr (D >= 64) {
        if (shared) {
            auto srow_out = attn_bwd_row_shared_kernel<E, D, kSW, kRowNS, true, SV>;
            auto scol_out = attn_bwd_col_shared_kernel<E, D, kSW, kColNS, true, SV>;
            if (e = allow_smem(srow_out, RowShape::smem); e != hipSuccess) return e;
            if (e = allow_smem(scol_out, ColShape::smem); e != hipSuccess) return e;
            hipLaunchKernelGGL(srow_out, grid_shared, dim3(64 * kSW), RowShape::smem, st, o);
            hipLaunchKernelGGL(scol_out, grid_shared, dim3(64 * kSW), ColShape::smem, st, o);
        }
    }
    // the two row passes share a launch when their grids are the same (attn_bwd_row_pair_kernel); the outer one then
    // waits for the outer column pass, which the inner one needs
    const bool rows_together = !shared && pair_out == pair_in;
    if (!shared) {
        if (!rows_together) hipLaunchKernelGGL(krow, attn_grid(a, Tp, pair_out), dim3(64 * kW), (row_smem<D, kW>()), st, o);
        hipLaunchKernelGGL(kcol_link, attn_grid(a, Tp, pair_out), dim3(64 * kW), (col_smem<D, kW, kRing>()), st, o);
    }

    // inner pass: X = K2, G = dR, K = K1, V = U
    AttnBwdP<E, SV> i{};
    i.x = caller_view<E, SV>(a, a.k2, a.lk2); i.g = dense_view<E, SV>(a, ws + l.dr); i.k = caller_view<E, SV>(a, a.k1, a.lk1);
    i.v = dense_view<E, SV>(a, ws + l.u);
    i.kp = (const E*)(ws + l.k1p1); i.vp = (const E*)(ws + l.up1); i.kp2 = (const E*)(ws + l.k1p2);
    i.xp = (const E*)(ws + l.k2p1); i.gp = (const E*)(ws + l.drp1);
    i.xp2 = (const E*)(ws + l.k2p2); i.gp2 = (const E*)(ws + l.drp2);
    i.lse2 = (const float*)(ws + l.lse1); i.delta = (const float*)(ws + l.delta1);
    i.BH = a.BH; i.H = a.H; i.T = a.T; i.Tp = Tp; i.alpha = a.alpha; i.causal = a.causal; i.k_diff = a.k_diff;
    i.pair = pair_in;
    i.addend = (const float*)(ws + l.dk2p); i.dx = (E*)a.dk2;
    i.dk = (E*)a.dk1; i.v1 = caller_view<E, SV>(a, a.v1, a.lv1); i.dv = (E*)a.dv1;
    if constexpr (D >= 64) {
        if (shared) {
            auto srow_in = attn_bwd_row_shared_kernel<E, D, kSW, kRowNS, false, SV>;
            auto scol_in = attn_bwd_col_shared_kernel<E, D, kSW, kColNS, false, SV>;
            if (e = allow_smem(srow_in, RowShape::smem); e != hipSuccess) return e;
            if (e = allow_smem(scol_in, ColShape::smem); e != hipSuccess) return e;
            hipLaunchKernelGGL(srow_in, grid_shared, dim3(64 * kSW), RowShape::smem, st, i);
            hipLaunchKernelGGL(scol_in, grid_shared, dim3(64 * kSW), ColShape::smem, st, i);
        }
    }
    if (!shared) {
        if (rows_together) {
            auto krow2 = attn_bwd_row_pair_kernel<E, D, kW, SV>;
            if (e = allow_smem(krow2, row_smem<D, kW>()); e != hipSuccess) return e;
            const dim3 g1 = attn_grid(a, Tp, pair_in);
            hipLaunchKernelGGL(krow2, dim3(g1.x, 2), dim3(64 * kW), (row_smem<D, kW>()), st, o, i);
        } else {
            hipLaunchKernelGGL(krow, attn_grid(a, Tp, pair_in), dim3(64 * kW), (row_smem<D, kW>()), st, i);
        }
        hipLaunchKernelGGL(kcol, attn_grid(a, Tp, pair_in), dim3(64 * kW), (col_smem<D, kW, kRing>()), st, i);
    }
    return hipGetLastError();
}

}  // namespace

bool mfma_dps_supported(int D, int dtype_is_16bit) { return dtype_is_16bit && (D == 32 || D == 64 || D == 128); }
size_t mfma_dps_fwd_workspace(int BH, int T, int D) { return layout(BH, T, D, false).total; }
size_t mfma_dps_bwd_workspace(int BH, int T, int D) { return layout(BH, T, D, true).total; }

// Waves per workgroup (they split the streamed tiles of an owner tile), measured at B*H = 32..64, bf16, forward /
// backward in us, (waves, paired) = (2, no) | (4, no) | (4, yes):  T=512: 29 / 100 | 32 / 118 | 31 / 115;
// T=1024: 42 / 137 | 39 / 145 | 38 / 142;  T=2048: 65 / 208 | 54 / 199 | 52 / 197;  T=4096: 112 / 351 | 84 / 309 | 81 / 308.
// Two waves at D = 128 (fewer partial results to merge); at D = 64 four waves from T = 2048 on, and from T = 1024 in
// the forward, or when the grid is too small to give every CU four workgroups of two waves.
static bool two_waves(const MfmaDpsArgs& a, bool backward) {
    if (a.D == 128) return true;
    if (a.D == 64 && knobs().dps_waves) return knobs().dps_waves == 2;
    const int workgroups = 8 * ((a.BH + 7) / 8) * ((a.T + 31) / 32);
    if (workgroups < 1024) return false;
    return a.T < (backward ? 2048 : 1024);
}

template <typename E, bool SV>
static hipError_t dps_fwd_typed(const MfmaDpsArgs& a, hipStream_t st) {
    if (a.D == 32) return run_fwd<E, 32, 4, SV>(a, st, false);
    if (a.D == 64) return two_waves(a, false) ? run_fwd<E, 64, 2, SV>(a, st, false) : run_fwd<E, 64, 4, SV>(a, st, false);
    if (a.D == 128) return run_fwd<E, 128, 2, SV>(a, st, false);
    return hipErrorInvalidValue;
}
template <typename E, bool SV>
static hipError_t dps_bwd_typed(const MfmaDpsArgs& a, hipStream_t st) {
    if (a.D == 32) return run_bwd<E, 32, 4, SV>(a, st);
    if (a.D == 64) return two_waves(a, true) ? run_bwd<E, 64, 2, SV>(a, st) : run_bwd<E, 64, 4, SV>(a, st);
    if (a.D == 128) return run_bwd<E, 128, 2, SV>(a, st);
    return hipErrorInvalidValue;
}

// a.H > 0: the caller's tensors are strided views (the kernels that take strides); otherwise the dense kernels
hipError_t mfma_dps_fwd(const MfmaDpsArgs& a, hipStream_t st) {
    if (a.H > 0) return a.is_bf16 ? dps_fwd_typed<__bf16, true>(a, st) : dps_fwd_typed<_Float16, true>(a, st);
    return a.is_bf16 ? dps_fwd_typed<__bf16, false>(a, st) : dps_fwd_typed<_Float16, false>(a, st);
}

hipError_t mfma_dps_bwd(const MfmaDpsArgs& a, hipStream_t st) {
    if (a.H > 0) return a.is_bf16 ? dps_bwd_typed<__bf16, true>(a, st) : dps_bwd_typed<_Float16, true>(a, st);
    return a.is_bf16 ? dps_bwd_typed<__bf16, false>(a, st) : dps_bwd_typed<_Float16, false>(a, st);
}

}  // namespace tritt
