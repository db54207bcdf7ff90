// Shared device helpers for the trittention HIP kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tritt {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct bf16_t {
    uint16_t bits;
};
using f16_t = _Float16;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t v) { return (float)v; }

// round-to-nearest-even fp32 -> bf16 (NaN kept quiet)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float v) { return (f16_t)v; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }
__device__ __forceinline__ float silu_grad_f(float x) {
    float s = 1.0f / (1.0f + __expf(-x));
    return s * (1.0f + x * (1.0f - s));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// One 64-row block of a row-major [T][D] tensor, transposed into dst[d][Tp] (rows past T become zeros), through
// an LDS tile so that both the reads (8 consecutive d of a row) and the writes (8 consecutive rows of a column)
// are whole 16-byte pieces: an element-wise transposed copy touches one cache line per lane and is bound by the
// address traffic of the vector memory path.  256 threads; `tile` holds 64 x (D + 2) elements; the caller
// synchronises the workgroup between transpose_load and transpose_store (and again before reusing the tile).
// SILU applies x -> SiLU(x) on the way and, with `rows` non-null, also stores the result row-major.
template <typename E, bool SILU>
__device__ __forceinline__ void transpose_load(const E* __restrict__ src, E* __restrict__ rows, E* tile, int j0, int T,
                                               int D, unsigned src_stride = 0 /* elements between rows of src; 0: D */) {
    typedef __attribute__((ext_vector_type(8))) E e8;
    const int ld = D + 2, cpr = D / 8;
    for (int idx = threadIdx.x; idx < 64 * cpr; idx += 256) {
        const int jj = idx / cpr, c = idx % cpr, j = j0 + jj;
        e8 x;
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (E)0.f;
        if (j < T) {
            x = *reinterpret_cast<const e8*>(src + (size_t)j * (src_stride ? src_stride : (unsigned)D) + c * 8);
            if (SILU) {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (E)silu_f((float)x[e]);
                if (rows) *reinterpret_cast<e8*>(rows + (size_t)j * D + c * 8) = x;
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) tile[jj * ld + c * 8 + e] = x[e];
    }
}
template <typename E>
__device__ __forceinline__ void transpose_store(E* __restrict__ dst, const E* tile, int j0, int Tp, int D) {
    typedef __attribute__((ext_vector_type(8))) E e8;
    const int ld = D + 2;
    for (int idx = threadIdx.x; idx < D * 8; idx += 256) {
        const int d = idx >> 3, cj = idx & 7;
        e8 y;
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = tile[(cj * 8 + e) * ld + d];
        *reinterpret_cast<e8*>(dst + (size_t)d * Tp + j0 + cj * 8) = y;
    }
}

// ---- XCD-aware order of a one-dimensional grid over (batch*head slice, tile) pairs -------------------------------
// Consecutive workgroup ids go to different XCDs (eight of them, each with its own L2), so workgroup id b works for
// XCD b % 8 and slot b / 8 of that XCD's list.  Whole groups of eight slices give every XCD its own slices (their keys
// and values stay in that XCD's L2), tiles in launch order 0 .. ntiles - 1 (callers map order 0 to their heaviest tile).
// The B*H % 8 slices left over would keep only some XCDs busy (B*H = 4: half the chip), so their (slice, tile) pairs are
// dealt out over all eight XCDs instead, ahead of the whole groups (their light tiles then overlap the groups' heavy
// ones; the end of the grid is light tiles either way).  xcd_slots = list length per XCD = grid size / 8.
__host__ __device__ inline int xcd_slots(int BH, int ntiles) {
    return (BH >> 3) * ntiles + (((BH & 7) * ntiles + 7) >> 3);
}
// false: a padding workgroup (the left-over pairs do not fill the last slot of every XCD)
__device__ __forceinline__ bool xcd_tile(int BH, int ntiles, int slot, int xcd, int& bh, int& order) {
    const int gf = BH >> 3, r = BH & 7, rem_slots = (r * ntiles + 7) >> 3;
    if (slot < rem_slots) {
        const int idx = slot * 8 + xcd;
        bh = gf * 8 + idx % r;
        order = idx / r;
        return idx < r * ntiles;
    }
    slot -= rem_slots;
    bh = (slot % gf) * 8 + xcd;
    order = slot / gf;
    return true;
}

// ---- 64-bit fixed-point gradient accumulators (backward kernels whose workgroups add shares of one gradient
// element to a common sum; integer addition is associative, so the sums do not depend on the order of arrival).
// The scale is a power of two chosen per (batch, head) slice from the largest finite |dO| of that slice,
// 2^e <= max|dO| < 2^(e+1): a share v is added as round(v * 2^(bias - e)), so the accumulators resolve steps of
// 2^-bias relative to the incoming gradient whatever its magnitude (loss scaling, mean-reduced losses) and cover
// sums up to 2^(63 - bias) times it.  Scaling dO by a power of two scales every gradient by exactly that power.
// The producer of the scale leaves kScaleParts partial maxima per slice (bit patterns of |dO|, non-finite values
// skipped); every consumer joins them.  A share that is not finite, or too large for the accumulator, cannot be
// represented in it: it sets a bit in the row's poison word instead, and the kernel that converts the
// accumulators writes NaN for that row of that gradient (the fp32 sums these accumulators stand in for would
// have been non-finite as well).
constexpr int kScaleParts = 8;
enum : unsigned { kPoisonDK1 = 1, kPoisonDU = 2, kPoisonDK2 = 4, kPoisonDV2 = 8, kPoisonDQ = 16 };

__device__ __forceinline__ unsigned finite_abs_bits(float v) {
    const unsigned b = __float_as_uint(v) & 0x7fffffffu;
    return b < 0x7f800000u ? b : 0u;
}
// exponent field f of the scale 2^(f - 127) of slice bh.  UNIFORM: bh is the same in every lane of the wave (the
// result is then kept in a scalar register); the kernels that convert the accumulators walk elements of several
// slices in one wave and pass false.
template <bool UNIFORM = true>
__device__ __forceinline__ int fixed_scale_field(const unsigned* __restrict__ parts, int bh, int bias) {
    const uint4 a = reinterpret_cast<const uint4*>(parts)[bh * 2], b = reinterpret_cast<const uint4*>(parts)[bh * 2 + 1];
    unsigned m = max(max(max(a.x, a.y), max(a.z, a.w)), max(max(b.x, b.y), max(b.z, b.w)));
    if (UNIFORM) m = __builtin_amdgcn_readfirstlane(m);
    const int f = bias + 254 - (int)(m >> 23);  // bias - (exponent - 127) + 127
    return min(max(f, 1), 254);
}
__device__ __forceinline__ float fixed_scale_value(int field) { return __uint_as_float((unsigned)field << 23); }
__device__ __forceinline__ double fixed_scale_inverse(int field) {
    return __longlong_as_double((long long)(1023 + 127 - field) << 52);
}
// One share of a common sum.  fscale == 0: the accumulator is fp32 (float atomics; non-finite values propagate by
// themselves).  poison_row: the poison word of the element's row; bit: which gradient.
__device__ __forceinline__ void shared_add(void* acc, size_t idx, float v, float fscale, unsigned* poison_row,
                                           unsigned bit) {
    if (fscale != 0.f) {
        const float x = v * fscale;
        if (!(fabsf(x) < 9.0e18f)) {  // NaN, Inf or beyond 2^63
            atomicOr(poison_row, bit);
            return;
        }
        atomicAdd(reinterpret_cast<unsigned long long*>(acc) + idx, (unsigned long long)__float2ll_rn(x));
    } else {
        unsafeAtomicAdd(reinterpret_cast<float*>(acc) + idx, v);
    }
}
// block-wide maximum of the finite |x| bit patterns of `count` 16-byte pieces (E8 = 8 elements of E, or 4 floats)
// starting at src; every thread of the 256-thread block returns the same value; `red` = 4 words of LDS
// (row_pieces > 0: the pieces form rows of row_pieces pieces that lie `pitch` elements apart)
template <typename E>
__device__ __forceinline__ unsigned block_absmax_bits(const E* __restrict__ src, size_t count, unsigned* red,
                                                      unsigned row_pieces = 0, unsigned pitch = 0) {
    constexpr int PER = 16 / sizeof(E);
    typedef __attribute__((ext_vector_type(PER))) E ev;
    unsigned m = 0;
    for (size_t i = threadIdx.x; i < count; i += 256) {
        const size_t at = row_pieces ? (i / row_pieces) * pitch + (i % row_pieces) * PER : i * PER;
        const ev x = *reinterpret_cast<const ev*>(src + at);
#pragma unroll
        for (int e = 0; e < PER; ++e) m = max(m, finite_abs_bits((float)x[e]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, off, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    return max(max(red[0], red[1]), max(red[2], red[3]));
}

// Window parameters of the triple-dot causal mask, expressed for a "staged"
// index a and an "owner" index b (a = j, b = k in the natural orientation):
//   valid  <=>  a<=q, b<=q, q<=a+wa, q<=b+wb, b<=a+lab, a<=b+rab
struct TdpMask {
    int causal;
    int wa, wb, lab, rab;
};

__device__ __forceinline__ bool tdp_valid(const TdpMask& m, int q, int a, int b) {
    if (!m.causal) return true;
    return (a <= q) & (b <= q) & (q <= a + m.wa) & (q <= b + m.wb) & (b <= a + m.lab) & (a <= b + m.rab);
}

}  // namespace tritt
