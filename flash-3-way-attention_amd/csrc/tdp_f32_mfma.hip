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
#include "tdp_f32_tiles.hpp"

namespace tritt {
namespace {

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
    F32BwdParams<E> r0, r1;
    int roles, rounds;
    if (hipError_t e = tile0_prepare<E, D>(a, st, r0, r1, roles, rounds); e != hipSuccess) return e;
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
