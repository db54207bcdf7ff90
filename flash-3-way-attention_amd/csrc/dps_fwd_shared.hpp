// Included by dps_mfma.hip inside namespace tritt::{anonymous}: the forward attention-with-bias kernel in the
// shape of a flash-attention forward.  A workgroup of kW waves owns 32 * kW query-like rows, one tile of 32 per wave,
// and walks the streamed 32-row tiles once for all of them: a tile's packed operands (K in packing P1, the values in
// packing P2, the per-key bias) are fetched straight into an LDS ring by direct-to-LDS loads, kNS - 1 tiles ahead,
// and every wave reads its MFMA operands from there.  Against one owner tile per workgroup with the waves splitting
// the streamed tiles, the operand fetches from L2 drop by kW and no partial softmax has to be merged.
//
// A packed tile is CH = 2 * D / 16 blocks of 64 lanes x 16 B, each exactly what one operand read of a wave wants, so
// the blocks land in LDS as they lie in memory and lane i reads 16 B at block + 16 i: conflict-free without a swizzle.
// Every wave fetches CH / kW blocks of each tile and its own copy of the bias (64 floats by one 4-byte load per
// lane), so all waves issue the same number of loads per tile and one wait count serves them all.
#pragma once

template <int D, int kW, int kNS>
struct FwdSharedShape {
    static constexpr int KS = D / 16, DT = D / 32;
    static constexpr int CH = 2 * KS;      // 1 KB blocks of a streamed tile: KS of K, then 2 DT of the values
    static constexpr int LW = CH / kW;     // blocks a wave fetches per tile
    static constexpr int kStage = CH * 1024 + kW * 256;             // bytes: blocks, then a bias copy per wave
    static constexpr int kOutTile = D * kLdr * 4;                   // a wave's output tile on its way out
    static constexpr size_t smem = kNS * kStage > kW * kOutTile ? kNS * kStage : kW * kOutTile;
    static_assert(CH % kW == 0, "the blocks of a tile are dealt out evenly to the waves");
};

// BIAS: keys carry a bias (the outer pass); otherwise no bias is fetched (the inner pass).
// With a multiplier (p.mul) every 16-bit output is the product out * mul, so `out` is for passes without one.
template <typename E, int D, int kW, int kNS, bool BIAS, bool SV>
__global__ __launch_bounds__(64 * kW, 2) void attn_fwd_shared_kernel(AttnFwdP<E, SV> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using S = FwdSharedShape<D, kW, kNS>;
    constexpr int KS = S::KS, DT = S::DT, LW = S::LW;
    constexpr int kLoads = LW + (BIAS ? 1 : 0);  // vector-memory operations per wave and tile
    extern __shared__ __align__(16) char smem_raw[];

    const int n_owner = (p.Tp / 32 + kW - 1) / kW;
    int bh, tile;
    if (!block_to_tile(p.BH, n_owner, bh, tile)) return;
    const int r0 = (n_owner - 1 - tile) * 32 * kW;  // longest rows first
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T, Tp = p.Tp;
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp, vb = (size_t)bh * Tp;
    const char* KP = reinterpret_cast<const char*>(uniform_ptr(p.kp + tb));
    const char* VP2 = reinterpret_cast<const char*>(uniform_ptr(p.vp2 + tb));
    const char* BP = BIAS ? reinterpret_cast<const char*>(uniform_ptr(p.bias + vb)) : nullptr;
    const int rw0 = r0 + 32 * wave, r = rw0 + n;
    const int2 at = slice_at<SV>(bh, p.H);

    // streamed tiles of the workgroup and of this wave's rows
    const int last_row = min(T - 1, r0 + 32 * kW - 1);
    const int t_first = p.causal ? max(0, r0 - p.k_diff) / 32 : 0;
    const int t_last = (p.causal ? last_row : T - 1) / 32;
    const int tw_first = p.causal ? max(0, rw0 - p.k_diff) / 32 : 0;
    const int tw_last = rw0 < T ? (p.causal ? min(T - 1, rw0 + 31) : T - 1) / 32 : -1;

    // tile t -> ring slot `slot` (tiles past t_last are fetched as t_last once more: the wait counts stay fixed and
    // nothing reads those slots)
    auto fetch = [&](int t, int slot) {
        char* dst = smem_raw + slot * S::kStage;
        const int tt = min(t, t_last);
#pragma unroll
        for (int j = 0; j < LW; ++j) {
            const int c = wave * LW + j;  // block of the tile
            const char* src = c < KS ? KP + ((size_t)tt * KS + c) * 1024 : VP2 + ((size_t)tt * KS + (c - KS)) * 1024;
            direct_load_16(src, lane * 16, dst + c * 1024);
        }
        if constexpr (BIAS)
            direct_load_4(BP, (unsigned)min(tt * 32 + lane, Tp - 1) * 4, dst + S::CH * 1024 + wave * 256);
    };
#pragma unroll
    for (int j = 0; j < kNS - 1; ++j) fetch(t_first + j, j);

    v8 xb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xb[ks] = ld8<E>(p.x.row(at, min(r, T - 1), T, D) + 16 * ks + 8 * g);
    // the rows must have arrived before the loop: a wait for them placed inside it would also wait for the
    // tiles fetched ahead, every time round
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xb[ks]));

    // the multiplier of the lane's outputs (4 consecutive d per register quad), fetched now so that the epilogue does
    // not wait for it
    typedef __attribute__((ext_vector_type(4))) E v4;
    const size_t row_off = base + (size_t)min(r, T - 1) * D;
    v4 mv[DT][4];
    if (p.mul) {
        const E* __restrict__ mul_row = p.mul.row(at, min(r, T - 1), T, D);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) mv[dt][q4] = *reinterpret_cast<const v4*>(mul_row + 32 * dt + 8 * q4 + 4 * g);
    }

    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    int slot = 0;
    for (int t = t_first; t <= t_last; ++t) {
        // tile t has landed (this wave's part: all but the loads of the kNS - 2 tiles after it; the others' parts:
        // the barrier), and every wave is done with tile t - 1, whose slot the next fetch overwrites
        barrier_keep_loads<kLoads * (kNS - 2)>();
        fetch(t + kNS - 1, slot == 0 ? kNS - 1 : slot - 1);
        const char* st = smem_raw + slot * S::kStage;
        slot = slot == kNS - 1 ? 0 : slot + 1;
        if (t < tw_first || t > tw_last) continue;  // outside this wave's band
        const int a0 = t * 32;
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            s = M::mma(*reinterpret_cast<const v8*>(st + ks * 1024 + lane * 16), xb[ks], s);
        float b[16];
        if constexpr (BIAS) {
            const float* sb = reinterpret_cast<const float*>(st + S::CH * 1024 + wave * 256);
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const float4 v = *reinterpret_cast<const float4*>(sb + 16 * h + 8 * g + 4 * c);
                    b[8 * h + 4 * c] = v.x; b[8 * h + 4 * c + 1] = v.y; b[8 * h + 4 * c + 2] = v.z; b[8 * h + 4 * c + 3] = v.w;
                }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) b[i] = 0.f;
        }
        // only tiles on an edge of the band (or past the end of the sequence) need the element-wise mask
        const bool edge = (a0 + 31 >= T) || (p.causal && ((a0 + 31 > rw0) || (rw0 + 31 - a0 > p.k_diff)));
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
        float tmax = fmaxf(sv[0], sv[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) tmax = fmaxf(fmaxf(tmax, sv[i]), sv[i + 1]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        // the reference maximum is raised lazily, as in attn_fwd_mfma_kernel
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
                acc[dt] = M::mma(*reinterpret_cast<const v8*>(st + (KS + dt * 2 + kk) * 1024 + lane * 16), pb[kk], acc[dt]);
    }
    l += __shfl_xor(l, 32, 64);
    // the tiles fetched past the end have landed and every wave has read its last tile: the ring becomes the
    // waves' output tiles
    barrier_keep_loads<0>();

    if (rw0 >= Tp) return;  // no row of this wave exists, not even as padding of the packed outputs
    const float inv = 1.0f / l;
    if (g == 0 && r < T) p.lse[(size_t)bh * p.lse_stride + r] = (m + fast_log2(l)) * p.lse_scale;
    float* sT = reinterpret_cast<float*>(smem_raw + wave * S::kOutTile);  // [D][kLdr], this wave's alone
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const int d0 = 32 * dt + 8 * q4 + 4 * g;  // registers 4 q4 .. 4 q4 + 3 are d0 .. d0 + 3 of row r
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = acc[dt][4 * q4 + j] * inv;
            if (p.out_f32 && r < T) *reinterpret_cast<float4*>(p.out_f32 + row_off + d0) = make_float4(o[0], o[1], o[2], o[3]);
            if (p.mul) {
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] *= (float)mv[dt][q4][j];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) sT[(d0 + j) * kLdr + n] = r < T ? o[j] : 0.f;
        }
    // the tile leaves in whole 16-byte pieces of each layout (wave-local: no barrier)
    const int rr = lane & 31, row = rw0 + rr;
#pragma unroll
    for (int c = g; c < D / 8; c += 2) {
        const int d0 = 8 * c;
        v8 wv;
#pragma unroll
        for (int j = 0; j < 8; ++j) wv[j] = (E)sT[(d0 + j) * kLdr + rr];
        const size_t off = base + (size_t)row * D + d0;
        if (row < T) {
            if (p.out) *reinterpret_cast<v8*>(p.out + off) = wv;
            if (p.outm) *reinterpret_cast<v8*>(p.outm + off) = wv;
        }
        if (p.outm_p1) *reinterpret_cast<v8*>(p.outm_p1 + tb + p1_index<D>(row, d0)) = wv;
    }
    if (p.outm_p2) {
#pragma unroll
        for (int j = 0; j < DT * 2; ++j) {  // piece (d-tile, half) = j of the wave's tile, lane's 8 rows of column d
            const int dt = j >> 1, kk = j & 1, r8 = kk * 16 + g * 8, d = dt * 32 + n;
            v8 y;
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = (E)sT[d * kLdr + r8 + e];
            *reinterpret_cast<v8*>(p.outm_p2 + tb + ((size_t)(((rw0 >> 5) * DT + dt) * 2 + kk) * 64 + lane) * 8) = y;
        }
    }
}
