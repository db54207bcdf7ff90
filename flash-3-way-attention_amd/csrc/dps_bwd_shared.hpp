// Included by dps_mfma.hip inside namespace tritt::{anonymous}: the two backward attention-with-bias kernels in the
// shape of dps_fwd_shared.hpp.  A workgroup of kW waves owns 32 * kW rows (row kernel: query-like rows; column
// kernel: key-like rows), one tile of 32 per wave, and walks the streamed 32-row tiles once for all of them; a
// tile's packed operands land in an LDS ring by direct-to-LDS loads, kNS - 1 tiles ahead, and every wave reads its
// MFMA operands (and the tile's per-row vectors) from there.  No partial result crosses waves, so nothing is merged;
// the operand fetches from L2 drop by kW.  Taken by large grids (see run_bwd).
#pragma once

template <int D, int kW, int kNS, int kTensors>
struct BwdSharedShape {
    static constexpr int KS = D / 16, DT = D / 32;
    static constexpr int CH = kTensors * KS;  // 1 KB blocks of a streamed tile (every packed tensor is KS of them)
    static constexpr int LW = CH / kW;        // blocks a wave fetches per tile
    static constexpr int kVec = 2;            // per-row vectors of a tile (bias | LSE, Delta), a copy per wave each
    static constexpr int kStage = CH * 1024 + kVec * kW * 256;
    static constexpr int kOutTile = D * kLdr * 4;  // a wave's output tile on its way out
    static constexpr size_t smem = kNS * kStage > kW * kOutTile ? kNS * kStage : kW * kOutTile;
    static_assert(CH % kW == 0, "the blocks of a tile are dealt out evenly to the waves");
};

// ------------------------------------------------------------------------------ rows: dX
// streamed per tile: K in packing P1 (scores), V in packing P1 (dP), K in packing P2 (dX), the per-key bias
template <typename E, int D, int kW, int kNS, bool BIAS, bool SV>
__global__ __launch_bounds__(64 * kW, 2) void attn_bwd_row_shared_kernel(AttnBwdP<E, SV> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using S = BwdSharedShape<D, kW, kNS, 3>;
    constexpr int KS = S::KS, DT = S::DT, LW = S::LW;
    constexpr int kLoads = LW + (BIAS ? 1 : 0);
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
    const char* VP = reinterpret_cast<const char*>(uniform_ptr(p.vp + tb));
    const char* KP2 = reinterpret_cast<const char*>(uniform_ptr(p.kp2 + tb));
    const char* BP = BIAS ? reinterpret_cast<const char*>(uniform_ptr(p.bias + vb)) : nullptr;
    const int rw0 = r0 + 32 * wave, r = rw0 + n, rc = min(r, T - 1);
    const float scale_log2 = p.alpha * kLog2e;
    const int2 at = slice_at<SV>(bh, p.H);

    const int last_row = min(T - 1, r0 + 32 * kW - 1);
    const int t_first = p.causal ? max(0, r0 - p.k_diff) / 32 : 0;
    const int t_last = (p.causal ? last_row : T - 1) / 32;
    const int tw_first = p.causal ? max(0, rw0 - p.k_diff) / 32 : 0;
    const int tw_last = rw0 < T ? (p.causal ? min(T - 1, rw0 + 31) : T - 1) / 32 : -1;

    // the blocks this wave fetches of every tile: where they start in tile 0 and where they go in a ring slot (picked
    // once: chosen inside the loop, the three sources become a table in scratch memory)
    const char* gsrc[LW];
    int gdst[LW];
#pragma unroll
    for (int j = 0; j < LW; ++j) {
        const int c = __builtin_amdgcn_readfirstlane(wave * LW + j), which = c / KS, blk = c % KS;
        gsrc[j] = uniform_ptr((which == 0 ? KP : which == 1 ? VP : KP2) + blk * 1024);
        gdst[j] = c * 1024;
    }
    // tile t -> ring slot (tiles past t_last are fetched as t_last once more: the wait counts stay fixed)
    auto fetch = [&](int t, int slot) {
        char* dst = smem_raw + __builtin_amdgcn_readfirstlane(slot * S::kStage);
        const int tt = __builtin_amdgcn_readfirstlane(min(t, t_last));
#pragma unroll
        for (int j = 0; j < LW; ++j) direct_load_16(uniform_ptr(gsrc[j] + (size_t)tt * KS * 1024), lane * 16, dst + gdst[j]);
        if constexpr (BIAS) direct_load_4(BP, (unsigned)min(tt * 32 + lane, Tp - 1) * 4, dst + S::CH * 1024 + wave * 256);
    };
#pragma unroll
    for (int j = 0; j < kNS - 1; ++j) fetch(t_first + j, j);

    v8 xb[KS], gb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        xb[ks] = ld8<E>(p.x.row(at, rc, T, D) + 16 * ks + 8 * g);
        gb[ks] = ld8<E>(p.g.row(at, rc, T, D) + 16 * ks + 8 * g);
    }
    float lse2 = p.lse2[vb + rc], dl = p.delta[vb + rc];
    // everything the loop reads from registers has arrived before it starts: a wait placed inside the loop would also
    // wait for the tiles fetched ahead
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xb[ks]), "+v"(gb[ks]));
    asm volatile("" : "+v"(lse2), "+v"(dl));

    f32x16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;

    int slot = 0;
    for (int t = t_first; t <= t_last; ++t) {
        barrier_keep_loads<kLoads * (kNS - 2)>();  // tile t has landed for everyone; tile t - 1's slot is free
        fetch(t + kNS - 1, slot == 0 ? kNS - 1 : slot - 1);
        const char* st = smem_raw + slot * S::kStage;
        slot = slot == kNS - 1 ? 0 : slot + 1;
        if (t < tw_first || t > tw_last) continue;  // outside this wave's band
        const int a0 = t * 32;
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = 0.f;
            dp[i] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = M::mma(*reinterpret_cast<const v8*>(st + ks * 1024 + lane * 16), xb[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = M::mma(*reinterpret_cast<const v8*>(st + (KS + ks) * 1024 + lane * 16), gb[ks], dp);
        float b[16];
        if constexpr (BIAS) {
            tile_vector(reinterpret_cast<const float*>(st + S::CH * 1024 + wave * 256), g, b);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) b[i] = 0.f;
        }
        // only tiles on an edge of the band (or past the end of the sequence) need the element-wise mask
        const bool edge = (a0 + 31 >= T) || (rw0 + 31 >= T) || (p.causal && ((a0 + 31 > rw0) || (rw0 + 31 - a0 > p.k_diff)));
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
        v8 dsb[2];
        pack16<E>(ds, dsb);
        // dX^T[d][r] += K^T[d][a] dS^T[a][r]
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
                acc[dt] = M::mma(*reinterpret_cast<const v8*>(st + (2 * KS + dt * 2 + kk) * 1024 + lane * 16), dsb[kk], acc[dt]);
    }
    barrier_keep_loads<0>();  // the ring becomes the waves' output tiles

    if (rw0 >= T) return;
    float* sT = reinterpret_cast<float*>(smem_raw + wave * S::kOutTile);  // [D][kLdr], this wave's alone
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sT[(32 * dt + c_row(g, i)) * kLdr + n] = acc[dt][i];
    const int rr = lane & 31, row = rw0 + rr;
    if (row >= T) return;
#pragma unroll
    for (int c = g; c < D / 8; c += 2) {
        const int d0 = 8 * c;
        const size_t off = base + (size_t)row * D + d0;
        v8 ov;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float v = sT[(d0 + j) * kLdr + rr] * p.alpha;
            if (p.addend) v += p.addend[off + j];
            ov[j] = (E)v;
        }
        *reinterpret_cast<v8*>(p.dx + off) = ov;
    }
}

// ------------------------------------------------------------------------------ columns: dK, dV, dbias
// streamed per tile: X and G in packing P1 (scores, dP) and in packing P2 (dK, dV), the rows' LSE and Delta
// (D = 128: two owner operands and four accumulators of 32 registers each leave no room for 256 registers a lane)
template <typename E, int D, int kW, int kNS, bool LINK, bool SV>
__global__ __launch_bounds__(64 * kW, (D <= 64 ? 2 : 1)) void attn_bwd_col_shared_kernel(AttnBwdP<E, SV> p) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using S = BwdSharedShape<D, kW, kNS, 4>;
    constexpr int KS = S::KS, DT = S::DT, LW = S::LW;
    constexpr int kLoads = LW + 2;
    extern __shared__ __align__(16) char smem_raw[];

    const int n_owner = (p.Tp / 32 + kW - 1) / kW;
    int bh, tile;
    if (!block_to_tile(p.BH, n_owner, bh, tile)) return;
    const int c0 = tile * 32 * kW;  // lowest key rows are the longest
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T, Tp = p.Tp;
    const size_t base = (size_t)bh * T * D, tb = (size_t)bh * D * Tp, vb = (size_t)bh * Tp;
    const char* XP = reinterpret_cast<const char*>(uniform_ptr(p.xp + tb));
    const char* GP = reinterpret_cast<const char*>(uniform_ptr(p.gp + tb));
    const char* XP2 = reinterpret_cast<const char*>(uniform_ptr(p.xp2 + tb));
    const char* GP2 = reinterpret_cast<const char*>(uniform_ptr(p.gp2 + tb));
    const char* LP = reinterpret_cast<const char*>(uniform_ptr(p.lse2 + vb));
    const char* DP = reinterpret_cast<const char*>(uniform_ptr(p.delta + vb));
    const int cw0 = c0 + 32 * wave, a = cw0 + n, ac = min(a, T - 1);
    const float scale_log2 = p.alpha * kLog2e;
    const int2 at = slice_at<SV>(bh, p.H);

    // streamed row tiles of the workgroup and of this wave's keys
    const int t_first = p.causal ? c0 / 32 : 0;
    const int t_last = (p.causal ? (int)min((long)T - 1, (long)c0 + 32 * kW - 1 + p.k_diff) : T - 1) / 32;
    const int tw_first = p.causal ? cw0 / 32 : 0;
    const int tw_last = cw0 < T ? (p.causal ? (int)min((long)T - 1, (long)cw0 + 31 + p.k_diff) : T - 1) / 32 : -1;

    // the blocks this wave fetches of every tile (see the row kernel)
    const char* gsrc[LW];
    int gdst[LW];
#pragma unroll
    for (int j = 0; j < LW; ++j) {
        const int c = __builtin_amdgcn_readfirstlane(wave * LW + j), which = c / KS, blk = c % KS;
        gsrc[j] = uniform_ptr((which == 0 ? XP : which == 1 ? GP : which == 2 ? XP2 : GP2) + blk * 1024);
        gdst[j] = c * 1024;
    }
    auto fetch = [&](int t, int slot) {
        char* dst = smem_raw + __builtin_amdgcn_readfirstlane(slot * S::kStage);
        const int tt = __builtin_amdgcn_readfirstlane(min(t, t_last));
#pragma unroll
        for (int j = 0; j < LW; ++j) direct_load_16(uniform_ptr(gsrc[j] + (size_t)tt * KS * 1024), lane * 16, dst + gdst[j]);
        const unsigned voff = (unsigned)min(tt * 32 + lane, Tp - 1) * 4;
        direct_load_4(LP, voff, dst + S::CH * 1024 + wave * 256);
        direct_load_4(DP, voff, dst + S::CH * 1024 + (kW + wave) * 256);
    };
#pragma unroll
    for (int j = 0; j < kNS - 1; ++j) fetch(t_first + j, j);

    v8 kb[KS], vbv[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kb[ks] = ld8<E>(p.k.row(at, ac, T, D) + 16 * ks + 8 * g);
        vbv[ks] = ld8<E>(p.v.row(at, ac, T, D) + 16 * ks + 8 * g);
    }
    float ba = p.bias ? p.bias[vb + ac] : 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(kb[ks]), "+v"(vbv[ks]));
    asm volatile("" : "+v"(ba));

    f32x16 acck[DT], accv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acck[dt][i] = 0.f;
            accv[dt][i] = 0.f;
        }
    float db = 0.f;

    int slot = 0;
    for (int t = t_first; t <= t_last; ++t) {
        barrier_keep_loads<kLoads * (kNS - 2)>();
        fetch(t + kNS - 1, slot == 0 ? kNS - 1 : slot - 1);
        const char* st = smem_raw + slot * S::kStage;
        slot = slot == kNS - 1 ? 0 : slot + 1;
        if (t < tw_first || t > tw_last) continue;
        const int r0 = t * 32;
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
        tile_vector(reinterpret_cast<const float*>(st + S::CH * 1024 + wave * 256), g, ls);
        tile_vector(reinterpret_cast<const float*>(st + S::CH * 1024 + (kW + wave) * 256), g, dl);
        const bool edge = (r0 + 31 >= T) || (cw0 + 31 >= T) || (p.causal && ((cw0 + 31 > r0) || (r0 + 31 - cw0 > p.k_diff)));
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
        // dK^T[d][a] += X^T[d][r] dS[r][a];  dV^T[d][a] += G^T[d][r] P[r][a]
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                acck[dt] = M::mma(*reinterpret_cast<const v8*>(st + (2 * KS + dt * 2 + kk) * 1024 + lane * 16), dsb[kk], acck[dt]);
                accv[dt] = M::mma(*reinterpret_cast<const v8*>(st + (3 * KS + dt * 2 + kk) * 1024 + lane * 16), pb[kk], accv[dt]);
            }
    }
    db += __shfl_xor(db, 32, 64);
    barrier_keep_loads<0>();  // the ring becomes the waves' output tiles

    if (cw0 >= Tp) return;  // no key of this wave exists, not even as padding of the packed outputs
    float* sT = reinterpret_cast<float*>(smem_raw + wave * S::kOutTile);  // [D][kLdr], this wave's alone
    const int aa = lane & 31, row = cw0 + aa;
    // ---- dK
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sT[(32 * dt + c_row(g, i)) * kLdr + n] = acck[dt][i];
    if (row < T) {
#pragma unroll
        for (int c = g; c < D / 8; c += 2) {
            const int d0 = 8 * c;
            const size_t off = base + (size_t)row * D + d0;
            float o[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = sT[(d0 + j) * kLdr + aa] * p.alpha;
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
    // ---- dV (the wave's LDS tile is read and written by this wave alone, in program order)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) sT[(32 * dt + c_row(g, i)) * kLdr + n] = accv[dt][i];
    float part = 0.f;
#pragma unroll
    for (int c = g; c < D / 8; c += 2) {
        const int d0 = 8 * c;
        const size_t off = base + (size_t)row * D + d0;
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = sT[(d0 + j) * kLdr + aa];
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
            // dR in packing P2 wants 8 consecutive rows of one column in a piece: through the LDS tile once more, below
#pragma unroll
            for (int j = 0; j < 8; ++j) sT[(d0 + j) * kLdr + aa] = (float)dr[j];
        }
    }
    if constexpr (LINK) {
        // delta1 = rowsum(dR R) - dbias: the two lanes of a row hold its pieces of either parity
        part += __shfl_xor(part, 32, 64);
        if (g == 0) p.delta1[vb + row] = row < T ? part - db : 0.f;
#pragma unroll
        for (int j = 0; j < DT * 2; ++j) {  // piece (d-tile, half) = j of the wave's tile, lane's 8 rows of column d
            const int dt = j >> 1, kk = j & 1, r8 = kk * 16 + g * 8, d = dt * 32 + n;
            v8 y;
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = (E)sT[d * kLdr + r8 + e];
            *reinterpret_cast<v8*>(p.dr_p2 + tb + ((size_t)(((cw0 >> 5) * DT + dt) * 2 + kk) * 64 + lane) * 8) = y;
        }
    }
}
