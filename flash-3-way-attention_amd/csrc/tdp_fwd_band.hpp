// Triple-dot-product trittention forward for NARROW windowed causal masks (gfx950, 16-bit tensors):
// the band-resident kernel.  Included by tdp_fwd_mfma.hip (FwdParams, kLazyThreshold).
//
// Under a windowed mask a query q only sees keys j in [q - wa, q] and k in [q - wb, q].  When the
// windows are narrow, every key row a tile of 32 queries can touch (at most max(wa, wb) + 32 + 31 rows
// of K1, U^T, K2 and V2) fits in LDS at once.  The workgroup loads that band ONCE, synchronises once,
// and from then on its eight waves run independently with no barrier and no global load: each wave
// walks its four queries one after another, per query the k-tiles of 32 inside [q - wb, q], per k-tile
// the 32-key steps of j inside the band of that tile.  Same formulation as the streaming kernel (virtual
// rows (q, k), transposed scores, P fed back as the A operand); what changes is that a k-tile of a narrow
// band has only a handful of steps, so everything per k-tile is kept cheap:
//   * FAST sweep first (P = exp2(S), reference 0, no maximum tracking); a wave whose sweep left the
//     safe exponent range repeats it by itself with the CAREFUL online softmax.
//   * masks of the k-j band come from a table in LDS: the pattern of a 32x32 step depends only on
//     (first key j - first key k), and at most four such offsets straddle an edge of the band; the
//     table holds them in the MFMA C layout (0 or -3e4), read as the C operand of the score product.
//     Steps cut by j <= q or j >= q - wa, and k-tiles cut by the k window, are masked element-wise.
//   * with reference 0 everywhere the merge of a k-tile into the running output needs no maximum, no
//     rescaling and no row weights (masked rows have P = 0 exactly): O += V2[k] (.) Tv[(q,k)].
#pragma once

namespace tritt {

constexpr int kBandQ = 32;  // queries per workgroup: 8 waves x 4

// rows of the resident band: everything queries q0 .. q0+31 can touch (q0 is a multiple of 32, and so is the
// first resident row)
inline int band_rows(int wa, int wb) { return ((wa > wb ? wa : wb) + 31) / 32 * 32 + kBandQ; }

template <int D>
constexpr size_t band_smem_bytes(int nr) {
    return sizeof(uint16_t) * ((size_t)3 * nr * (D + 8) + (size_t)D * (nr + 8)) + sizeof(float) * (kBandQ * D + 8 * 32 + 5 * 16 * 64);
}

template <typename E, int D, bool MV = false>
__global__ __launch_bounds__(512, 2) void tdp_fwd_band_kernel(FwdParams<E> p, int NR) {
    using M = Mma<E>;
    using v8 = typename M::v8;
    using v2 = typename M::v2;
    constexpr int KS = D / 16, DT = D / 32, LDK = D + 8;
    const int LDU = NR + 8;

    extern __shared__ __align__(16) char smem[];
    E* sK1 = reinterpret_cast<E*>(smem);  // [NR][LDK]
    E* sK2 = sK1 + NR * LDK;
    E* sV2 = sK2 + NR * LDK;
    E* sUT = sV2 + NR * LDK;               // [D][LDU]
    float* sQ = reinterpret_cast<float*>(sUT + D * LDU);  // [32][D]  Q * alpha*log2(e), fp32
    float* sW = sQ + kBandQ * D;                                // [8][32] per-wave scratch
    float* sTab = sW + 8 * 32;  // [5 slots][4][64 lanes][4]  band masks in the MFMA C layout; slot 4: zeros

    int bh, order;
    if (!xcd_tile(p.BH, p.nqt, blockIdx.x >> 3, blockIdx.x & 7, bh, order)) return;
    const int qt = p.nqt - 1 - order;

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.T;
    const size_t base = (size_t)bh * T * D;  // of the outputs
    const size_t in_base = (size_t)(bh / p.H) * p.in_sb + (size_t)(bh % p.H) * p.in_sh;
    const unsigned in_st = p.in_st;
    const E* __restrict__ Q = p.q + in_base;
    const int wa = p.wa, wb = p.wb, lab = p.lab, rab = p.rab;
    const int q0 = qt * kBandQ;
    const int rlo = max(0, q0 - max(wa, wb)) & ~31;  // first resident key row

    // ---- load the band ---------------------------------------------------------------------------
    {
        auto slice = [&](const E* t, const TensorAt& at) {
            return MV ? t + (size_t)(bh / p.H) * at.sb + (size_t)(bh % p.H) * at.sh : t + in_base;
        };
        const E* __restrict__ K1 = slice(p.k1, p.at_k1);
        const E* __restrict__ K2 = slice(p.k2, p.at_k2);
        const E* __restrict__ V2 = slice(p.v2, p.at_v2);
        const unsigned st_k1 = MV ? p.at_k1.st : in_st, st_k2 = MV ? p.at_k2.st : in_st, st_v2 = MV ? p.at_v2.st : in_st;
        const E* __restrict__ UT = p.ut + (size_t)bh * D * p.Tp;
        const int row_chunks = NR * (D / 8);
        for (int c = tid; c < row_chunks; c += 512) {
            const int r = c / (D / 8), ch = c % (D / 8);
            const unsigned row = (unsigned)min(rlo + r, T - 1);
            const uint4 a = *reinterpret_cast<const uint4*>(K1 + (size_t)(row * st_k1) + ch * 8);
            const uint4 b = *reinterpret_cast<const uint4*>(K2 + (size_t)(row * st_k2) + ch * 8);
            const uint4 v = *reinterpret_cast<const uint4*>(V2 + (size_t)(row * st_v2) + ch * 8);
            *reinterpret_cast<uint4*>(sK1 + r * LDK + ch * 8) = a;
            *reinterpret_cast<uint4*>(sK2 + r * LDK + ch * 8) = b;
            *reinterpret_cast<uint4*>(sV2 + r * LDK + ch * 8) = v;
        }
        const int ut_chunks = D * (NR / 8);
        for (int c = tid; c < ut_chunks; c += 512) {
            const int d = c / (NR / 8), cj = c % (NR / 8);
            const int j0 = rlo + cj * 8;
            uint4 u = {0u, 0u, 0u, 0u};
            if (j0 + 8 <= p.Tp) u = *reinterpret_cast<const uint4*>(UT + (size_t)d * p.Tp + j0);
            *reinterpret_cast<uint4*>(sUT + d * LDU + cj * 8) = u;
        }
    }
    for (int idx = tid; idx < kBandQ * D; idx += 512) {
        const int r = idx / D, d = idx % D;
        sQ[idx] = (float)Q[(size_t)((unsigned)min(q0 + r, T - 1) * in_st) + d] * p.scale_log2;
    }
    // ---- band mask table: slot -> offset m = (jb - k0) / 32 ----------------------------------------
    const int mlo = -((lab + 31) / 32), mhi = (rab + 31) / 32;
    if (tid < 320) {
        const int sl = tid >> 6, m = sl < 2 ? mlo + sl : mhi - (sl - 2);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int dlt = 32 * m + key_of(g, i) - n;  // j - k
            sTab[((sl * 4 + i / 4) * 64 + lane) * 4 + (i % 4)] = (sl == 4 || (dlt >= -lab && dlt <= rab)) ? 0.f : -3.0e4f;
        }
    }
    __syncthreads();
    // from here on the waves never meet again

    float* sWw = sW + wave * 32;
    const int krow_off = key_of_row(n);
    auto rows_of = [&](float v, float (&out)[16]) {
        if (g == 0) sWw[n] = v;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float4 f4 = *reinterpret_cast<const float4*>(sWw + 8 * b + 4 * g);
            out[4 * b] = f4.x; out[4 * b + 1] = f4.y; out[4 * b + 2] = f4.z; out[4 * b + 3] = f4.w;
        }
        __builtin_amdgcn_wave_barrier();
    };

    for (int qi = 0; qi < kBandQ / 8; ++qi) {
        const int q = q0 + wave + 8 * qi;  // interleaved: the waves' loads stay even at the start of a sequence
        if (q >= T) break;
        const float* sQw = sQ + (wave + 8 * qi) * D;

        float Mrun = -INFINITY, Lrun = 0.f, Orun[DT];  // Lrun, Orun: per-lane partial sums
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) Orun[dt] = 0.f;

        // k >= q - wb, and some j with q - wa <= j <= k + rab
        const int kt_a = max(0, max(q - wb, q - wa - rab)) / 32, kt_b = q / 32;
        for (int kt = kt_a; kt <= kt_b; ++kt) {
            const int k0 = kt * 32, k = k0 + n;
            // window of keys j of the virtual row (q, k); empty: hi < lo
            int wlo = max(q - wa, k - lab), whi = min(q, k + rab);
            if (k > q || q > k + wb || whi < wlo) { wlo = 0; whi = -1; }
            const bool kval = whi >= 0;
            // all 32 rows of the tile are inside the k window
            const bool rows_clean = (k0 + 31 <= q) && (q <= k0 + wb);
            const int jlo_t = max(0, max(q - wa, k0 - lab)), jhi_t = min(q, k0 + 31 + rab);
            const int jb_lo = jlo_t & ~31;
            if (jlo_t > jhi_t) continue;  // no (j, k) of this tile is inside the band of q

            v8 bq[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v8 kv = *reinterpret_cast<const v8*>(sK2 + (k0 - rlo + n) * LDK + ks * 16 + g * 8);
                const float* qp = sQw + ks * 16 + g * 8;
                const float4 qa = *reinterpret_cast<const float4*>(qp), qb = *reinterpret_cast<const float4*>(qp + 4);
                const float qf[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
                v8 r;
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const v2 pr = M::pack((float)kv[e] * qf[e], (float)kv[e + 1] * qf[e + 1]);
                    r[e] = pr[0];
                    r[e + 1] = pr[1];
                }
                bq[ks] = r;
            }

            f32x16 acc[DT];
            float mref = 0.f, lsum = 0.f;
            auto clear = [&] {
                mref = 0.f;
                lsum = 0.f;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
            };
            auto value_product = [&](const v8 (&pa)[2], int jb) {
                const E* utp = sUT + n * LDU + (jb - rlo) + g * 8;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        acc[dt] = M::mma(pa[h], *reinterpret_cast<const v8*>(utp + dt * 32 * LDU + h * 16), acc[dt]);
            };

            // ---- FAST sweep ---------------------------------------------------------------------
            // C operand of the score product = the mask, all of it additive: the k-j band from the table
            // (slot 4: all zeros), a per-lane penalty for rows outside the k window, and, on the steps the
            // limits j <= q / j >= q - wa cut through, an element-wise one.  The first step starts the
            // value accumulators from a zero C operand instead of cleared registers.
            const float row_pen = kval ? 0.f : -3.0e4f;
            auto fast_step = [&](int jb, auto first_tag) {
                constexpr bool FIRST = decltype(first_tag)::value;
                const E* k1p = sK1 + (jb - rlo + krow_off) * LDK + g * 8;
                const int m = (jb - k0) >> 5;
                const bool partial = 32 * m - 31 < -lab || 32 * m + 31 > rab;  // straddles an edge of the band
                const int sl = !partial ? 4 : (m - mlo < 2) ? m - mlo : 2 + (mhi - m);
                f32x16 s;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const float4 f4 = *reinterpret_cast<const float4*>(sTab + ((sl * 4 + b) * 64 + lane) * 4);
                    s[4 * b] = f4.x; s[4 * b + 1] = f4.y; s[4 * b + 2] = f4.z; s[4 * b + 3] = f4.w;
                }
                if (!rows_clean) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] += row_pen;
                }
                if (jb + 31 > q || jb < q - wa) {
                    const int lo = q - wa - jb - 8 * g, span = wa;  // valid: 0 <= key_of(0, i) - lo <= wa
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] = ((unsigned)(key_of(0, i) - lo) <= (unsigned)span) ? s[i] : -3.0e4f;
                }
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) s = M::mma(*reinterpret_cast<const v8*>(k1p + ks * 16), bq[ks], s);
                v8 pa[2];
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const v2 pr = M::pack(fast_exp2(s[h * 8 + e]), fast_exp2(s[h * 8 + e + 1]));
                        lsum = M::add_pair(pr, lsum);
                        pa[h][e] = pr[0];
                        pa[h][e + 1] = pr[1];
                    }
                const E* utp = sUT + n * LDU + (jb - rlo) + g * 8;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    f32x16 c;
                    if constexpr (FIRST) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) c[i] = 0.f;
                    } else {
                        c = acc[dt];
                    }
                    c = M::mma(pa[0], *reinterpret_cast<const v8*>(utp + dt * 32 * LDU), c);
                    acc[dt] = M::mma(pa[1], *reinterpret_cast<const v8*>(utp + dt * 32 * LDU + 16), c);
                }
            };
            mref = 0.f;
            lsum = 0.f;
            fast_step(jb_lo, std::true_type{});
            for (int jb = jb_lo + 32; jb <= jhi_t; jb += 32) fast_step(jb, std::false_type{});
            bool fast_ok;
            {
                // P <= its row sum, so a row sum inside this range keeps the value accumulators finite as well
                const float lk = lsum + __shfl_xor(lsum, 32, 64);
                fast_ok = !__any(kval && !(lk > fast_row_sum_floor<E>() && lk < 1e25f));
            }
            if (!fast_ok) {
                // ---- CAREFUL sweep: online softmax, reference raised lazily; a row may meet its first
                // valid key late, until then its reference sits at a finite floor
                clear();
                bool started = false;
                for (int jb = jb_lo; jb <= jhi_t; jb += 32) {
                    const E* k1p = sK1 + (jb - rlo + krow_off) * LDK + g * 8;
                    f32x16 s;
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) s = M::mma(*reinterpret_cast<const v8*>(k1p + ks * 16), bq[ks], s);
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int j = jb + key_of(g, i);
                        s[i] = (j >= wlo && j <= whi) ? s[i] : -INFINITY;
                    }
                    float mx = fmaxf(s[0], s[1]);
#pragma unroll
                    for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
                    const bool begin = !started;
                    started = true;
                    if (begin || __any(mx - mref > kLazyThreshold)) {
                        const float rmax = fmaxf(fmaxf(mx, __shfl_xor(mx, 32, 64)), -1.0e30f);
                        const float newref = begin ? rmax : fmaxf(rmax, mref);
                        const float f = fast_exp2(mref - newref);
                        mref = newref;
                        if (!begin) {
                            lsum *= f;
                            float fr[16];
                            rows_of(f, fr);
#pragma unroll
                            for (int i = 0; i < 16; ++i)
#pragma unroll
                                for (int dt = 0; dt < DT; ++dt) acc[dt][i] *= fr[i];
                        }
                    }
                    v8 pa[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const v2 pr = M::pack(fast_exp2(s[h * 8 + e] - mref), fast_exp2(s[h * 8 + e + 1] - mref));
                            lsum = M::add_pair(pr, lsum);
                            pa[h][e] = pr[0];
                            pa[h][e + 1] = pr[1];
                        }
                    value_product(pa, jb);
                }
            }

            // ---- merge the 32 virtual rows (q, k) into the running output ---------------------------
            const E* v2p = sV2 + (k0 - rlo) * LDK + n;
            if (fast_ok && (Mrun == 0.f || Mrun == -INFINITY)) {
                // everything so far is relative to reference 0 and masked rows hold exact zeros
                Mrun = 0.f;
                Lrun += lsum;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    float part = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; ++i) part += (float)v2p[c_row(g, i) * LDK + dt * 32] * acc[dt][i];
                    Orun[dt] += part;
                }
            } else {
                float mt = kval ? mref : -INFINITY;
#pragma unroll
                for (int off = 16; off > 0; off >>= 1) mt = fmaxf(mt, __shfl_xor(mt, off, 64));
                const float mnew = fmaxf(Mrun, mt);
                const float f = (mnew == -INFINITY) ? 1.f : fast_exp2(Mrun - mnew);
                const float w = kval ? fast_exp2(mref - mnew) : 0.f;
                Lrun = Lrun * f + w * lsum;
                Mrun = mnew;
                float wr[16];
                rows_of(w, wr);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    float part = 0.f;
#pragma unroll
                    for (int i = 0; i < 16; ++i) part += wr[i] * (float)v2p[c_row(g, i) * LDK + dt * 32] * acc[dt][i];
                    Orun[dt] = Orun[dt] * f + part;
                }
            }
        }

        // ---- this query is done --------------------------------------------------------------------
        float L = Lrun;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) L += __shfl_xor(L, off, 64);
        const float inv = 1.0f / L;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const float o = (Orun[dt] + __shfl_xor(Orun[dt], 32, 64)) * inv;
            if (g == 0) p.o[base + (size_t)q * D + dt * 32 + n] = (E)o;
        }
        if (lane == 0) p.lse[(size_t)bh * T + q] = (Mrun + fast_log2(L)) * kLn2;
    }
}

}  // namespace tritt
