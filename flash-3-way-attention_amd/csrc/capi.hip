// C ABI of libtrittention_hip.so: argument checks, scratch layout, dispatch.
// Declarations and the contract of each entry point: include/trittention_hip.h.
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>
#include "../../include/trittention_hip.h"

#include "common.hpp"
#include "kernels.hpp"

namespace tritt {

namespace {
std::atomic<int> g_knobs[TRITT_TUNE_COUNT_];
std::once_flag g_knobs_once;
void init_knobs() {
    std::call_once(g_knobs_once, [] {
        if (const char* e = getenv("TRITT_FWD_SPLITS")) g_knobs[TRITT_TUNE_FWD_SPLITS] = atoi(e);
        if (const char* e = getenv("TRITT_FWD_BAND")) g_knobs[TRITT_TUNE_FWD_BAND] = atoi(e) == 0 ? -1 : 0;
        if (const char* e = getenv("TRITT_BWD_SPLITS")) g_knobs[TRITT_TUNE_BWD_SPLITS] = atoi(e);
        if (const char* e = getenv("TRITT_BWD128_VARIANT"))
            g_knobs[TRITT_TUNE_BWD128_WAVES] = strcmp(e, "w4") == 0 ? 4 : strcmp(e, "w8") == 0 ? 8 : 0;
        if (const char* e = getenv("TRITT_F32_VALU")) g_knobs[TRITT_TUNE_F32_VALU] = atoi(e) != 0 ? 1 : 0;
    });
}
}  // namespace

Knobs knobs() {
    init_knobs();
    return Knobs{g_knobs[TRITT_TUNE_FWD_SPLITS].load(), g_knobs[TRITT_TUNE_FWD_BAND].load(),
                 g_knobs[TRITT_TUNE_BWD_SPLITS].load(), g_knobs[TRITT_TUNE_BWD128_WAVES].load(),
                 g_knobs[TRITT_TUNE_F32_VALU].load(), g_knobs[TRITT_TUNE_DPS_WAVES].load(),
                 g_knobs[TRITT_TUNE_DPS_PAIR].load(), g_knobs[TRITT_TUNE_DPS_SHARED].load()};
}

hipError_t ensure_dynamic_smem(const void* kernel, size_t bytes) {
    struct Entry {
        int device;
        const void* kernel;
        size_t bytes;
    };
    static std::mutex mutex;
    static std::vector<Entry> done;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mutex);
    for (Entry& en : done)
        if (en.device == device && en.kernel == kernel) {
            if (en.bytes >= bytes) return hipSuccess;
            e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
            if (e == hipSuccess) en.bytes = bytes;
            return e;
        }
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) done.push_back({device, kernel, bytes});
    return e;
}

namespace {

// Bump allocator over the caller's workspace; with base == nullptr it only measures.
struct Arena {
    char* base;
    size_t off = 0;
    explicit Arena(void* b) : base(static_cast<char*>(b)) {}
    template <typename T>
    T* take(size_t count) {
        off = (off + 255) & ~size_t(255);
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += count * sizeof(T);
        return p;
    }
    size_t bytes() const { return (off + 255) & ~size_t(255); }
};

size_t elem_size(int dtype) { return dtype == TRITT_F32 ? 4 : 2; }

int check_common(int B, int H, int T, int D, int dtype) {
    if (B <= 0 || H <= 0 || T <= 0) return TRITT_ERR_INVALID;
    if (dtype != TRITT_F32 && dtype != TRITT_BF16 && dtype != TRITT_F16) return TRITT_ERR_INVALID;
    if (D != 8 && D != 16 && D != 32 && D != 64 && D != 128) return TRITT_ERR_HEAD_DIM;
    if ((long long)B * H > 65535) return TRITT_ERR_INVALID;
    if ((long long)B * H * T > 0x7fffffffLL) return TRITT_ERR_INVALID;  // row indices are 32-bit; element offsets are not
    return TRITT_OK;
}

// An empty batch, head set or sequence: nothing to compute, no pointer is touched.
bool empty_problem(int B, int H, int T) { return B >= 0 && H >= 0 && T >= 0 && (B == 0 || H == 0 || T == 0); }

// ---------------------------------------------------------------- elementwise helpers
template <typename T, bool SILU>
__global__ __launch_bounds__(256) void to_f32_kernel(const T* __restrict__ src, float* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float v = to_float(src[i]);
        dst[i] = SILU ? silu_f(v) : v;
    }
}

// dst = src (* SiLU'(v1) when v1 != nullptr), converted to T
template <typename T>
__global__ __launch_bounds__(256) void from_f32_kernel(const float* __restrict__ src, const T* __restrict__ v1,
                                                       T* __restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        float v = src[i];
        if (v1) v *= silu_grad_f(to_float(v1[i]));
        dst[i] = from_float<T>(v);
    }
}

// delta[row] = sum_d a[row, d] * b[row, d]   (one wave per row)
template <typename T>
__global__ __launch_bounds__(256) void rowdot_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                     float* __restrict__ out, int rows, int D) {
    const int lane = threadIdx.x & 63;
    // grid-stride over rows: the grid is capped, and rows may be close to 2^31
    for (long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += (long long)gridDim.x * 4) {
        float part = 0.f;
        for (int d = lane; d < D; d += 64) part += to_float(a[(size_t)row * D + d]) * to_float(b[(size_t)row * D + d]);
        part = wave_sum(part);
        if (lane == 0) out[row] = part;
    }
}

unsigned ew_grid(size_t n) {
    size_t g = (n + 255) / 256;
    return (unsigned)(g > 8192 ? 8192 : g);
}

template <bool SILU>
void to_f32(const void* src, float* dst, size_t n, int dtype, hipStream_t st) {
    if (dtype == TRITT_F32)
        hipLaunchKernelGGL((to_f32_kernel<float, SILU>), dim3(ew_grid(n)), dim3(256), 0, st, (const float*)src, dst, n);
    else if (dtype == TRITT_BF16)
        hipLaunchKernelGGL((to_f32_kernel<bf16_t, SILU>), dim3(ew_grid(n)), dim3(256), 0, st, (const bf16_t*)src, dst, n);
    else
        hipLaunchKernelGGL((to_f32_kernel<f16_t, SILU>), dim3(ew_grid(n)), dim3(256), 0, st, (const f16_t*)src, dst, n);
}

void from_f32(const float* src, const void* v1, void* dst, size_t n, int dtype, hipStream_t st) {
    if (dtype == TRITT_F32)
        hipLaunchKernelGGL(from_f32_kernel<float>, dim3(ew_grid(n)), dim3(256), 0, st, src, (const float*)v1, (float*)dst, n);
    else if (dtype == TRITT_BF16)
        hipLaunchKernelGGL(from_f32_kernel<bf16_t>, dim3(ew_grid(n)), dim3(256), 0, st, src, (const bf16_t*)v1, (bf16_t*)dst, n);
    else
        hipLaunchKernelGGL(from_f32_kernel<f16_t>, dim3(ew_grid(n)), dim3(256), 0, st, src, (const f16_t*)v1, (f16_t*)dst, n);
}

void rowdot(const void* a, const void* b, float* out, int rows, int D, int dtype, hipStream_t st) {
    const long long blocks = ((long long)rows + 3) / 4;
    dim3 grid((unsigned)(blocks > 65536 ? 65536 : blocks));
    if (dtype == TRITT_F32)
        hipLaunchKernelGGL(rowdot_kernel<float>, grid, dim3(256), 0, st, (const float*)a, (const float*)b, out, rows, D);
    else if (dtype == TRITT_BF16)
        hipLaunchKernelGGL(rowdot_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)a, (const bf16_t*)b, out, rows, D);
    else
        hipLaunchKernelGGL(rowdot_kernel<f16_t>, grid, dim3(256), 0, st, (const f16_t*)a, (const f16_t*)b, out, rows, D);
}

// fp32 views of the five inputs: in place for fp32 tensors, scratch copies otherwise; u = SiLU(v1).
struct F32Inputs {
    const float *q, *k1, *k2, *u, *v2;
};
F32Inputs plan_inputs(Arena& ar, const void* q, const void* k1, const void* k2, const void* v2, size_t n, int dtype,
                      float** copies /* [4] scratch or null */, float** u) {
    F32Inputs r{};
    *u = ar.take<float>(n);
    r.u = *u;
    if (dtype == TRITT_F32) {
        r.q = (const float*)q; r.k1 = (const float*)k1; r.k2 = (const float*)k2; r.v2 = (const float*)v2;
        for (int i = 0; i < 4; ++i) copies[i] = nullptr;
    } else {
        for (int i = 0; i < 4; ++i) copies[i] = ar.take<float>(n);
        r.q = copies[0]; r.k1 = copies[1]; r.k2 = copies[2]; r.v2 = copies[3];
    }
    return r;
}
void fill_inputs(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, size_t n, int dtype,
                 float* const* copies, float* u, hipStream_t st) {
    to_f32<true>(v1, u, n, dtype, st);
    if (dtype != TRITT_F32) {
        to_f32<false>(q, copies[0], n, dtype, st);
        to_f32<false>(k1, copies[1], n, dtype, st);
        to_f32<false>(k2, copies[2], n, dtype, st);
        to_f32<false>(v2, copies[3], n, dtype, st);
    }
}

int clampw(int w, int T) { return w > T ? T : w; }

// The fp32 path has two sets of kernels: on the matrix cores (v_mfma_f32_32x32x2_f32; a workgroup per 32 queries)
// and on the vector ALUs (a wave per query: far more workgroups, the better shape for problems of a few tiles).
bool use_f32_mfma(int BH, int T, bool backward = false) {
    if (knobs().f32_valu) return false;
    // the backward deals the rounds of a tile out to workgroups when the tiles alone leave the chip idle
    return (long long)BH * ((T + 31) / 32) >= (backward ? 8 : 64);
}

// ---------------------------------------------------------------- triple-dot, fp32 VALU path
int tdp_fwd_generic(Arena& ar, bool run, const void* q, const void* k1, const void* k2, const void* v1,
                    const void* v2, void* o, float* lse, int B, int H, int T, int D, int dtype, float alpha,
                    int causal, int w1, int w2, int kl, int kr, hipStream_t st) {
    const size_t n = (size_t)B * H * T * D;
    float *copies[4], *u;
    F32Inputs in = plan_inputs(ar, q, k1, k2, v2, n, dtype, copies, &u);
    float* o32 = dtype == TRITT_F32 ? (float*)o : ar.take<float>(n);
    if (!run) return TRITT_OK;
    fill_inputs(q, k1, k2, v1, v2, n, dtype, copies, u, st);
    GenericTdpArgs a{};
    a.q = in.q; a.k1 = in.k1; a.k2 = in.k2; a.u = in.u; a.v2 = in.v2;
    a.o = o32; a.lse = lse;
    a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha;
    a.causal = causal; a.k1_window = w1; a.k2_window = w2; a.kk_left = kl; a.kk_right = kr;
    // fp32 on the matrix cores where a kernel exists (D = 32, 64), fp32 VALU kernels otherwise
    hipError_t e = (f32_mfma_tdp_supported(D) && use_f32_mfma(B * H, T)) ? f32_mfma_tdp_fwd(a, st) : generic_tdp_fwd(a, st);
    if (e != hipSuccess) return (int)e;
    if (dtype != TRITT_F32) from_f32(o32, nullptr, o, n, dtype, st);
    return (int)hipGetLastError();
}

int tdp_bwd_generic(Arena& ar, bool run, const void* q, const void* k1, const void* k2, const void* v1,
                    const void* v2, const void* o, const float* lse, const void* d_o, void* dq, void* dk1,
                    void* dk2, void* dv1, void* dv2, int B, int H, int T, int D, int dtype, float alpha, int causal,
                    int w1, int w2, int kl, int kr, hipStream_t st) {
    const size_t n = (size_t)B * H * T * D;
    float *copies[4], *u;
    F32Inputs in = plan_inputs(ar, q, k1, k2, v2, n, dtype, copies, &u);
    float* do32 = dtype == TRITT_F32 ? (float*)d_o : ar.take<float>(n);
    float* delta = ar.take<float>((size_t)B * H * T);
    float* du = ar.take<float>(n);
    // fp32 results: the caller's tensors when they are fp32, scratch otherwise; `spare` stands in for the
    // unwanted (null) half of a gradient pair whose other half is wanted (one kernel writes both halves)
    float *dq32 = (float*)dq, *dk132 = (float*)dk1, *dk232 = (float*)dk2, *dv232 = (float*)dv2;
    float* spare = nullptr;
    if (dtype != TRITT_F32) {
        dq32 = ar.take<float>(n); dk132 = ar.take<float>(n); dk232 = ar.take<float>(n); dv232 = ar.take<float>(n);
    } else {
        spare = ar.take<float>(n);
    }
    long long* fixed = f32_mfma_tdp_supported(D) ? ar.take<long long>(f32_mfma_tdp_bwd_scratch_elems(B * H, T, D)) : nullptr;
    // 16-bit tensors on the fp32 path: the output and the log-sum-exp are formed once more in fp32, because Delta =
    // rowsum(dO * O) from the stored 16-bit output carries that output's rounding, which nearly one-hot softmax
    // rows (large scores, first causal rows) turn into gradient errors far above it
    float* o32 = dtype != TRITT_F32 ? ar.take<float>(n) : nullptr;
    float* lse32 = dtype != TRITT_F32 ? ar.take<float>((size_t)B * H * T) : nullptr;
    if (!run) return TRITT_OK;
    const bool want_k2 = dk2 || dv2, want_k1 = dk1 || dv1;
    if (dtype == TRITT_F32) {
        if (want_k2 && !dk2) dk232 = spare;
        if (want_k2 && !dv2) dv232 = spare;
        if (want_k1 && !dk1) dk132 = spare;
    }
    fill_inputs(q, k1, k2, v1, v2, n, dtype, copies, u, st);
    if (dtype != TRITT_F32) to_f32<false>(d_o, do32, n, dtype, st);
    GenericTdpArgs a{};
    a.q = in.q; a.k1 = in.k1; a.k2 = in.k2; a.u = in.u; a.v2 = in.v2;
    a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha;
    a.causal = causal; a.k1_window = w1; a.k2_window = w2; a.kk_left = kl; a.kk_right = kr;
    const bool mfma32 = fixed && use_f32_mfma(B * H, T, true);
    if (o32) {
        a.o = o32; a.lse = lse32;
        hipError_t ef = (fixed && use_f32_mfma(B * H, T)) ? f32_mfma_tdp_fwd(a, st) : generic_tdp_fwd(a, st);
        if (ef != hipSuccess) return (int)ef;
        rowdot(do32, o32, delta, B * H * T, D, TRITT_F32, st);
        lse = lse32;
    } else {
        rowdot(d_o, o, delta, B * H * T, D, dtype, st);
    }
    a.lse_in = lse; a.d_o = do32; a.delta = delta;
    a.dq = dq ? dq32 : nullptr;
    a.dk2 = want_k2 ? dk232 : nullptr; a.dv2 = want_k2 ? dv232 : nullptr;
    a.dk1 = want_k1 ? dk132 : nullptr; a.du = want_k1 ? du : nullptr;
    hipError_t e = mfma32 ? f32_mfma_tdp_bwd(a, fixed, st) : generic_tdp_bwd(a, st);
    if (e != hipSuccess) return (int)e;
    if (dv1) from_f32(du, v1, dv1, n, dtype, st);
    if (dtype != TRITT_F32) {
        if (dq) from_f32(dq32, nullptr, dq, n, dtype, st);
        if (dk1) from_f32(dk132, nullptr, dk1, n, dtype, st);
        if (dk2) from_f32(dk232, nullptr, dk2, n, dtype, st);
        if (dv2) from_f32(dv232, nullptr, dv2, n, dtype, st);
    }
    return (int)hipGetLastError();
}

// ---------------------------------------------------------------- dot-product-sum
// fp32 path: the attention kernels on the fp32 matrix cores where they exist (D = 32, 64), else one lane per row on
// the vector ALUs; TRITT_TUNE_F32_VALU forces the latter
bool use_f32_mfma_dps(int D) { return !knobs().f32_valu && f32_mfma_dps_supported(D); }

int dps_fwd_impl(Arena& ar, bool run, const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                 void* o, float* lse, int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                 hipStream_t st) {
    const size_t n = (size_t)B * H * T * D, rows = (size_t)B * H * T;
    float *copies[4], *u;
    F32Inputs in = plan_inputs(ar, q, k1, k2, v2, n, dtype, copies, &u);
    float* o32 = dtype == TRITT_F32 ? (float*)o : ar.take<float>(n);
    DpsArgs a{};
    a.r = ar.take<float>(n);
    a.w = ar.take<float>(n);
    a.lse1 = ar.take<float>(rows);
    if (!run) return TRITT_OK;
    fill_inputs(q, k1, k2, v1, v2, n, dtype, copies, u, st);
    a.q = in.q; a.k1 = in.k1; a.k2 = in.k2; a.u = in.u; a.v2 = in.v2;
    a.o = o32; a.lse = lse;
    a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal; a.k_diff = k_diff;
    hipError_t e = use_f32_mfma_dps(D) ? f32_mfma_dps_fwd(a, st) : dps_fwd(a, st);
    if (e != hipSuccess) return (int)e;
    if (dtype != TRITT_F32) from_f32(o32, nullptr, o, n, dtype, st);
    return (int)hipGetLastError();
}

int dps_bwd_impl(Arena& ar, bool run, const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                 const void* o, const float* lse, const void* d_o, void* dq, void* dk1, void* dk2, void* dv1,
                 void* dv2, int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                 hipStream_t st) {
    const size_t n = (size_t)B * H * T * D, rows = (size_t)B * H * T;
    float *copies[4], *u;
    F32Inputs in = plan_inputs(ar, q, k1, k2, v2, n, dtype, copies, &u);
    float* do32 = dtype == TRITT_F32 ? (float*)d_o : ar.take<float>(n);
    DpsArgs a{};
    a.r = ar.take<float>(n); a.w = ar.take<float>(n); a.dw = ar.take<float>(n); a.dr = ar.take<float>(n);
    a.dk2_part = ar.take<float>(n);
    a.lse1 = ar.take<float>(rows); a.delta = ar.take<float>(rows);
    a.dlse1 = ar.take<float>(rows); a.delta1 = ar.take<float>(rows);
    float* du = ar.take<float>(n);
    float *dq32 = (float*)dq, *dk132 = (float*)dk1, *dk232 = (float*)dk2, *dv232 = (float*)dv2;
    if (dtype != TRITT_F32) {
        dq32 = ar.take<float>(n); dk132 = ar.take<float>(n); dk232 = ar.take<float>(n); dv232 = ar.take<float>(n);
    }
    // 16-bit tensors on the fp32 path: the output and the log-sum-exp are formed once more in fp32, as the triple-dot
    // path does: Delta = rowsum(dO * O) from the stored 16-bit output carries that output's rounding, which nearly
    // one-hot softmax rows (large scores) turn into gradient errors far above it
    float* o32 = dtype != TRITT_F32 ? ar.take<float>(n) : nullptr;
    float* lse32 = dtype != TRITT_F32 ? ar.take<float>(rows) : nullptr;
    if (!run) return TRITT_OK;
    fill_inputs(q, k1, k2, v1, v2, n, dtype, copies, u, st);
    if (dtype != TRITT_F32) to_f32<false>(d_o, do32, n, dtype, st);
    a.q = in.q; a.k1 = in.k1; a.k2 = in.k2; a.u = in.u; a.v2 = in.v2;
    a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal; a.k_diff = k_diff;
    if (o32) {
        a.o = o32; a.lse = lse32;
        hipError_t ef = use_f32_mfma_dps(D) ? f32_mfma_dps_fwd(a, st) : dps_fwd(a, st);
        if (ef != hipSuccess) return (int)ef;
        rowdot(do32, o32, a.delta, (int)rows, D, TRITT_F32, st);
        lse = lse32;
    } else {
        rowdot(d_o, o, a.delta, (int)rows, D, dtype, st);
    }
    a.lse = const_cast<float*>(lse); a.d_o = do32;
    a.dq = dq32; a.dk1 = dk132; a.dk2 = dk232; a.du = du; a.dv2 = dv232;
    hipError_t e = use_f32_mfma_dps(D) ? f32_mfma_dps_bwd(a, st) : dps_bwd(a, st);
    if (e != hipSuccess) return (int)e;
    from_f32(du, v1, dv1, n, dtype, st);
    if (dtype != TRITT_F32) {
        from_f32(dq32, nullptr, dq, n, dtype, st);
        from_f32(dk132, nullptr, dk1, n, dtype, st);
        from_f32(dk232, nullptr, dk2, n, dtype, st);
        from_f32(dv232, nullptr, dv2, n, dtype, st);
    }
    return (int)hipGetLastError();
}

// windows that cannot exclude any pair once j,k <= q holds
bool full_windows(int T, int causal, int w1, int w2, int kl, int kr) {
    return !causal || (w1 >= T - 1 && w2 >= T - 1 && kl >= T - 1 && kr >= T - 1);
}

// TRITT_FLAG_SPLIT_OPERANDS applies where the 16-bit MFMA kernels have a split-operand form
bool use_split(int D, int dtype, unsigned flags) {
    return (flags & TRITT_FLAG_SPLIT_OPERANDS) && !(flags & TRITT_FLAG_FORCE_GENERIC) &&
           mfma_tdp_split_supported(D, dtype != TRITT_F32);
}

bool use_mfma_fwd(int T, int D, int dtype, int causal, int w1, int w2, int kl, int kr, unsigned flags) {
    if (flags & TRITT_FLAG_FORCE_GENERIC) return false;
    (void)T; (void)causal; (void)w1; (void)w2; (void)kl; (void)kr;  // any mask: windows take the banded instantiation
    return mfma_tdp_fwd_supported(D, dtype != TRITT_F32);
}

bool use_mfma_bwd(int T, int D, int dtype, int causal, int w1, int w2, int kl, int kr, unsigned flags) {
    if (flags & TRITT_FLAG_FORCE_GENERIC) return false;
    (void)T; (void)causal; (void)w1; (void)w2; (void)kl; (void)kr;  // any mask: windows take the banded kernels
    return mfma_tdp_bwd_supported(D, dtype != TRITT_F32);
}

bool use_mfma_dps(int D, int dtype, unsigned flags) {
    if (flags & TRITT_FLAG_FORCE_GENERIC) return false;
    return mfma_dps_supported(D, dtype != TRITT_F32);
}

bool any_null(std::initializer_list<const void*> ps) {
    for (const void* p : ps)
        if (!p) return true;
    return false;
}

// the kernels move 16 bytes per lane: every [B,H,T,D] tensor must start on a 16-byte boundary
bool any_misaligned(std::initializer_list<const void*> ps) {
    for (const void* p : ps)
        if (reinterpret_cast<uintptr_t>(p) & 15) return true;
    return false;
}

// ---------------------------------------------------------------- strided views of the inputs
// A view is dense when it is the [B,H,T,D] layout itself (strides of dimensions of extent 1 never matter).
bool layout_dense(const tritt_layout* l, int B, int H, int T, int D) {
    if (!l) return true;
    return (T == 1 || l->stride_t == D) && (H == 1 || l->stride_h == (long long)T * D) &&
           (B == 1 || l->stride_b == (long long)H * T * D);
}
// 16-byte pieces must stay aligned: every stride a multiple of 16 bytes, none negative
int check_layout(const tritt_layout* l, int dtype) {
    if (!l) return TRITT_OK;
    const long long unit = 16 / (long long)elem_size(dtype);
    if (l->stride_b < 0 || l->stride_h < 0 || l->stride_t < 0) return TRITT_ERR_INVALID;
    if (l->stride_b % unit || l->stride_h % unit || l->stride_t % unit) return TRITT_ERR_INVALID;
    return TRITT_OK;
}
// a view's strides as the kernels take them (null: dense)
TensorAt tensor_at(const tritt_layout* l, int H, int T, int D) {
    if (!l) return dense_at(H, T, D);
    return TensorAt{l->stride_b, l->stride_h, (unsigned)(T == 1 ? D : l->stride_t)};
}
bool same_layout(const tritt_layout& a, const tritt_layout& b) {
    return a.stride_b == b.stride_b && a.stride_h == b.stride_h && a.stride_t == b.stride_t;
}

// Dense copies of up to six strided [B,H,T,D] views, one launch: blockIdx.y picks the view, a thread moves 16 bytes.
constexpr int kMaxViews = 6;
struct PackArgs {
    const char* src[kMaxViews];
    char* dst[kMaxViews];
    long long sb[kMaxViews], sh[kMaxViews], st[kMaxViews];  // bytes
    int H, T, pieces;                                       // pieces: 16-byte pieces per row
};
__global__ __launch_bounds__(256) void pack_kernel(PackArgs a, long long total) {
    const int v = blockIdx.y;
    const char* __restrict__ src = a.src[v];
    char* __restrict__ dst = a.dst[v];
    const long long sb = a.sb[v], sh = a.sh[v], st = a.st[v];
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int c = (int)(i % a.pieces);
        const long long row = i / a.pieces;
        const int t = (int)(row % a.T);
        const long long bh = row / a.T;
        const long long b = bh / a.H, h = bh % a.H;
        *reinterpret_cast<uint4*>(dst + i * 16) = *reinterpret_cast<const uint4*>(src + b * sb + h * sh + t * st + c * 16);
    }
}

// The plan of a strided call: which views are packed into the tail of the workspace, and what the dense entry point
// is then handed.  `base` null: measuring only.
struct Views {
    const void* ptr[kMaxViews];
    PackArgs pack;
    int jobs = 0;
    size_t bytes = 0;  // of the packed copies
};
void plan_view(Views& v, int slot, const void* src, const tritt_layout* l, bool keep, char* base, size_t n_bytes, int es) {
    v.ptr[slot] = src;
    if (keep) return;
    char* dst = base ? base + v.bytes : nullptr;
    v.bytes += (n_bytes + 255) & ~size_t(255);
    v.pack.src[v.jobs] = static_cast<const char*>(src);
    v.pack.dst[v.jobs] = dst;
    v.pack.sb[v.jobs] = l->stride_b * es; v.pack.sh[v.jobs] = l->stride_h * es; v.pack.st[v.jobs] = l->stride_t * es;
    ++v.jobs;
    v.ptr[slot] = dst;
}
void run_pack(Views& v, int B, int H, int T, int D, int dtype, hipStream_t st) {
    if (!v.jobs) return;
    v.pack.H = H; v.pack.T = T; v.pack.pieces = D * (int)elem_size(dtype) / 16;
    const long long total = (long long)B * H * T * v.pack.pieces;
    long long g = (total + 255) / 256;
    if (g > 4096) g = 4096;
    hipLaunchKernelGGL(pack_kernel, dim3((unsigned)g, v.jobs), dim3(256), 0, st, v.pack, total);
}
// every view of `src[count]` that is not dense gets a packed copy (layouts null: all dense)
int plan_all(Views& v, int first_slot, const void* const* src, const tritt_layout* layouts, int count, char* base, int B,
             int H, int T, int D, int dtype) {
    const size_t n_bytes = (size_t)B * H * T * D * elem_size(dtype);
    for (int i = 0; i < count; ++i) {
        const tritt_layout* l = layouts ? layouts + i : nullptr;
        if (int rc = check_layout(l, dtype); rc != TRITT_OK) return rc;
        plan_view(v, first_slot + i, src[i], l, layout_dense(l, B, H, T, D), base, n_bytes, (int)elem_size(dtype));
    }
    return TRITT_OK;
}
size_t round256(size_t x) { return (x + 255) & ~size_t(255); }

// Library-owned scratch of tritt_tdp_fwd_static_scratch: one copy per GPU the code object is loaded on, held
// until the process ends.  The name is a host-side stand-in; the device address comes from hipGetSymbolAddress.
static __device__ __align__(256) unsigned char scratch[TRITT_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device).
int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return TRITT_ERR_INVALID;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p || (reinterpret_cast<uintptr_t>(p) & 255)) return TRITT_ERR_INVALID;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TRITT_OK;
}

}  // namespace
}  // namespace tritt

using namespace tritt;

extern "C" {

int tritt_version(void) { return 200; }

int tritt_set_tuning(int knob, int value, int* previous) {
    if (knob < 0 || knob >= TRITT_TUNE_COUNT_) return TRITT_ERR_INVALID;
    init_knobs();
    const int old = g_knobs[knob].exchange(value);
    if (previous) *previous = old;
    return TRITT_OK;
}

const char* tritt_status_string(int status) {
    switch (status) {
        case TRITT_OK: return "ok";
        case TRITT_ERR_INVALID: return "invalid argument (null or misaligned pointer, non-positive size, negative window or unknown dtype)";
        case TRITT_ERR_HEAD_DIM: return "head dimension must be 8, 16, 32, 64 or 128";
        case TRITT_ERR_WORKSPACE: return "workspace missing or too small";
        case TRITT_ERR_UNSUPPORTED: return "requested implementation does not support this configuration";
        case TRITT_ERR_SCRATCH_LIMIT: return "problem needs more scratch than the library's static buffer holds";
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

// the fields of MfmaFwdArgs that describe the problem (no pointers)
static MfmaFwdArgs mfma_fwd_shape(int B, int H, int T, int D, int dtype, int causal, int k1_window, int k2_window,
                                  int kk_left, int kk_right, unsigned flags) {
    const int w1 = clampw(k1_window, T), w2 = clampw(k2_window, T), kl = clampw(kk_left, T), kr = clampw(kk_right, T);
    MfmaFwdArgs a{};
    a.BH = B * H; a.T = T; a.D = D; a.causal = causal ? 1 : 0;
    a.is_bf16 = dtype == TRITT_BF16;
    a.windowed = full_windows(T, causal, w1, w2, kl, kr) ? 0 : 1;
    a.k1_window = w1; a.k2_window = w2; a.kk_left = kl; a.kk_right = kr;
    a.split = use_split(D, dtype, flags) ? 1 : 0;
    return a;
}

size_t tritt_tdp_fwd_workspace_bytes(int B, int H, int T, int D, int dtype, int causal, int k1_window, int k2_window,
                                     int kk_left, int kk_right, unsigned flags) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_fwd(T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags))
        return mfma_tdp_fwd_workspace(mfma_fwd_shape(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags));
    Arena ar(nullptr);
    tdp_fwd_generic(ar, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, B, H, T, D, dtype, 0.f,
                    causal, k1_window, k2_window, kk_left, kk_right, nullptr);
    (void)flags;
    return ar.bytes();
}

int tritt_tdp_fwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, void* o, float* lse,
                  int B, int H, int T, int D, int dtype, float alpha, int causal, int k1_window, int k2_window,
                  int kk_left, int kk_right, void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o})) return TRITT_ERR_INVALID;
    if (causal && (k1_window < 0 || k2_window < 0 || kk_left < 0 || kk_right < 0)) return TRITT_ERR_INVALID;
    const int w1 = clampw(k1_window, T), w2 = clampw(k2_window, T), kl = clampw(kk_left, T), kr = clampw(kk_right, T);
    const bool mfma = use_mfma_fwd(T, D, dtype, causal, w1, w2, kl, kr, flags);
    if ((flags & TRITT_FLAG_FORCE_MFMA) && !mfma) return TRITT_ERR_UNSUPPORTED;
    // the caller sized `o` for two tensors: a path that writes one would leave the residual undefined
    if ((flags & TRITT_FLAG_SPLIT_OPERANDS) && !(mfma && use_split(D, dtype, flags))) return TRITT_ERR_UNSUPPORTED;
    const size_t need = tritt_tdp_fwd_workspace_bytes(B, H, T, D, dtype, causal, w1, w2, kl, kr, flags);
    if (need && (!workspace || workspace_bytes < need)) return TRITT_ERR_WORKSPACE;
    if (mfma) {
        MfmaFwdArgs a = mfma_fwd_shape(B, H, T, D, dtype, causal, w1, w2, kl, kr, flags);
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.lse = lse; a.ut = workspace;
        a.alpha = alpha;
        return (int)mfma_tdp_fwd(a, (hipStream_t)stream);
    }
    Arena ar(workspace);
    return tdp_fwd_generic(ar, true, q, k1, k2, v1, v2, o, lse, B, H, T, D, dtype, alpha, causal, w1, w2, kl, kr,
                           (hipStream_t)stream);
}

size_t tritt_static_scratch_bytes(void) { return TRITT_STATIC_SCRATCH_BYTES; }

int tritt_tdp_fwd_static_scratch(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, void* o,
                                 float* lse, int B, int H, int T, int D, int dtype, float alpha, int causal,
                                 int k1_window, int k2_window, int kk_left, int kk_right, unsigned flags,
                                 void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    const size_t need = tritt_tdp_fwd_workspace_bytes(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left,
                                                      kk_right, flags);
    if (need > TRITT_STATIC_SCRATCH_BYTES) return TRITT_ERR_SCRATCH_LIMIT;
    void* ws = nullptr;
    rc = static_scratch(&ws);
    if (rc != TRITT_OK) return rc;
    // every kernel of the forward writes the part of the scratch it later reads (the transposed SiLU(V1) copy
    // including its zero padding, the parts of a split forward): nothing has to be cleared between calls
    return tritt_tdp_fwd(q, k1, k2, v1, v2, o, lse, B, H, T, D, dtype, alpha, causal, k1_window, k2_window, kk_left,
                         kk_right, ws, TRITT_STATIC_SCRATCH_BYTES, flags, stream);
}

size_t tritt_tdp_bwd_workspace_bytes(int B, int H, int T, int D, int dtype, int causal, int k1_window, int k2_window,
                                     int kk_left, int kk_right, unsigned flags) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_bwd(T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags))
        return mfma_tdp_bwd_workspace(B * H, T, D, (flags & TRITT_FLAG_FLOAT_ATOMICS) == 0);
    Arena ar(nullptr);
    tdp_bwd_generic(ar, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                    nullptr, nullptr, nullptr, B, H, T, D, dtype, 0.f, causal, k1_window, k2_window, kk_left, kk_right,
                    nullptr);
    (void)flags;
    return ar.bytes();
}

int tritt_tdp_bwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, const void* o,
                  const float* lse, const void* d_o, void* dq, void* dk1, void* dk2, void* dv1, void* dv2, int B, int H,
                  int T, int D, int dtype, float alpha, int causal, int k1_window, int k2_window, int kk_left,
                  int kk_right, void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse, d_o})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o, d_o, dq, dk1, dk2, dv1, dv2})) return TRITT_ERR_INVALID;  // null is aligned
    if (!dq && !dk1 && !dk2 && !dv1 && !dv2) return TRITT_OK;  // no gradient wanted
    if (causal && (k1_window < 0 || k2_window < 0 || kk_left < 0 || kk_right < 0)) return TRITT_ERR_INVALID;
    const int w1 = clampw(k1_window, T), w2 = clampw(k2_window, T), kl = clampw(kk_left, T), kr = clampw(kk_right, T);
    const bool mfma = use_mfma_bwd(T, D, dtype, causal, w1, w2, kl, kr, flags);
    if ((flags & TRITT_FLAG_FORCE_MFMA) && !mfma) return TRITT_ERR_UNSUPPORTED;
    if ((flags & TRITT_FLAG_SPLIT_OPERANDS) && !(mfma && use_split(D, dtype, flags))) return TRITT_ERR_UNSUPPORTED;
    const size_t need = tritt_tdp_bwd_workspace_bytes(B, H, T, D, dtype, causal, w1, w2, kl, kr, flags);
    if (need && (!workspace || workspace_bytes < need)) return TRITT_ERR_WORKSPACE;
    if (mfma) {
        MfmaBwdArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.d_o = d_o; a.lse = lse;
        a.dq = dq; a.dk1 = dk1; a.dk2 = dk2; a.dv1 = dv1; a.dv2 = dv2; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0;
        a.is_bf16 = dtype == TRITT_BF16;
        a.windowed = full_windows(T, causal, w1, w2, kl, kr) ? 0 : 1;
        a.k1_window = w1; a.k2_window = w2; a.kk_left = kl; a.kk_right = kr;
        a.deterministic = (flags & TRITT_FLAG_FLOAT_ATOMICS) ? 0 : 1;
        a.split = use_split(D, dtype, flags) ? 1 : 0;
        return (int)mfma_tdp_bwd(a, (hipStream_t)stream);
    }
    Arena ar(workspace);
    return tdp_bwd_generic(ar, true, q, k1, k2, v1, v2, o, lse, d_o, dq, dk1, dk2, dv1, dv2, B, H, T, D, dtype, alpha,
                           causal, w1, w2, kl, kr, (hipStream_t)stream);
}

size_t tritt_dps_fwd_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_dps(D, dtype, flags)) return mfma_dps_fwd_workspace(B * H, T, D);
    Arena ar(nullptr);
    dps_fwd_impl(ar, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, B, H, T, D, dtype, 0.f, 1, T,
                 nullptr);
    (void)flags;
    return ar.bytes();
}

int tritt_dps_fwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, void* o, float* lse,
                  int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff, void* workspace,
                  size_t workspace_bytes, unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o})) return TRITT_ERR_INVALID;
    if (causal && k_diff < 0) return TRITT_ERR_INVALID;
    const bool mfma = use_mfma_dps(D, dtype, flags);
    if ((flags & TRITT_FLAG_FORCE_MFMA) && !mfma) return TRITT_ERR_UNSUPPORTED;
    const size_t need = tritt_dps_fwd_workspace_bytes(B, H, T, D, dtype, flags);
    if (!workspace || workspace_bytes < need) return TRITT_ERR_WORKSPACE;
    if (mfma) {
        MfmaDpsArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o_out = o; a.lse_out = lse; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0; a.k_diff = clampw(k_diff, T);
        a.is_bf16 = dtype == TRITT_BF16;
        return (int)mfma_dps_fwd(a, (hipStream_t)stream);
    }
    Arena ar(workspace);
    return dps_fwd_impl(ar, true, q, k1, k2, v1, v2, o, lse, B, H, T, D, dtype, alpha, causal, clampw(k_diff, T),
                        (hipStream_t)stream);
}

size_t tritt_dps_bwd_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_dps(D, dtype, flags)) return mfma_dps_bwd_workspace(B * H, T, D);
    Arena ar(nullptr);
    dps_bwd_impl(ar, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                 nullptr, nullptr, nullptr, B, H, T, D, dtype, 0.f, 1, T, nullptr);
    (void)flags;
    return ar.bytes();
}

int tritt_dps_bwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2, const void* o,
                  const float* lse, const void* d_o, void* dq, void* dk1, void* dk2, void* dv1, void* dv2, int B, int H,
                  int T, int D, int dtype, float alpha, int causal, int k_diff, void* workspace, size_t workspace_bytes,
                  unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse, d_o, dq, dk1, dk2, dv1, dv2})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o, d_o, dq, dk1, dk2, dv1, dv2})) return TRITT_ERR_INVALID;
    if (causal && k_diff < 0) return TRITT_ERR_INVALID;
    const bool mfma = use_mfma_dps(D, dtype, flags);
    if ((flags & TRITT_FLAG_FORCE_MFMA) && !mfma) return TRITT_ERR_UNSUPPORTED;
    const size_t need = tritt_dps_bwd_workspace_bytes(B, H, T, D, dtype, flags);
    if (!workspace || workspace_bytes < need) return TRITT_ERR_WORKSPACE;
    if (mfma) {
        MfmaDpsArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.d_o = d_o; a.lse_in = lse;
        a.dq = dq; a.dk1 = dk1; a.dk2 = dk2; a.dv1 = dv1; a.dv2 = dv2; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0; a.k_diff = clampw(k_diff, T);
        a.is_bf16 = dtype == TRITT_BF16;
        return (int)mfma_dps_bwd(a, (hipStream_t)stream);
    }
    Arena ar(workspace);
    return dps_bwd_impl(ar, true, q, k1, k2, v1, v2, o, lse, d_o, dq, dk1, dk2, dv1, dv2, B, H, T, D, dtype, alpha,
                        causal, clampw(k_diff, T), (hipStream_t)stream);
}

// ---------------------------------------------------------------- strided entry points
// The triple-dot forward on the 16-bit matrix-core path reads strided views in place: V1 through the SiLU / transpose
// pass, which takes its layout, the other four inside the main kernel (on one common layout, or each on its own: a
// second instantiation), when every row stride fits the kernels' 32-bit field.
static bool fwd_reads_in_place(const tritt_layout* l, int dtype, int T) {
    if (!l) return true;
    for (int i = 0; i < 5; ++i)
        // the kernels form row offsets in 32 bits; a row stride of 0 (a broadcast view) would read as "dense" in the
        // launch arguments
        if (check_layout(l + i, dtype) != TRITT_OK || (long long)T * l[i].stride_t > 0x7fffffffLL ||
            (T > 1 && l[i].stride_t == 0))
            return false;
    return true;
}

size_t tritt_tdp_fwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, int causal, int k1_window,
                                             int k2_window, int kk_left, int kk_right, unsigned flags,
                                             const tritt_layout* in_layouts) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    const size_t plain =
        round256(tritt_tdp_fwd_workspace_bytes(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags));
    if (use_mfma_fwd(T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags) &&
        fwd_reads_in_place(in_layouts, dtype, T))
        return plain;
    Views v;
    const void* none[5] = {};
    if (plan_all(v, 0, none, in_layouts, 5, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    return plain + v.bytes;
}

int tritt_tdp_fwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, void* o, float* lse, int B, int H, int T, int D, int dtype,
                          float alpha, int causal, int k1_window, int k2_window, int kk_left, int kk_right,
                          void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o})) return TRITT_ERR_INVALID;
    if (causal && (k1_window < 0 || k2_window < 0 || kk_left < 0 || kk_right < 0)) return TRITT_ERR_INVALID;
    for (int i = 0; in_layouts && i < 5; ++i)
        if ((rc = check_layout(in_layouts + i, dtype)) != TRITT_OK) return rc;
    const int w1 = clampw(k1_window, T), w2 = clampw(k2_window, T), kl = clampw(kk_left, T), kr = clampw(kk_right, T);
    const size_t plain = round256(tritt_tdp_fwd_workspace_bytes(B, H, T, D, dtype, causal, w1, w2, kl, kr, flags));
    const bool mfma = use_mfma_fwd(T, D, dtype, causal, w1, w2, kl, kr, flags);
    if (mfma && in_layouts && fwd_reads_in_place(in_layouts, dtype, T)) {
        if ((flags & TRITT_FLAG_SPLIT_OPERANDS) && !use_split(D, dtype, flags)) return TRITT_ERR_UNSUPPORTED;
        if (plain && (!workspace || workspace_bytes < plain)) return TRITT_ERR_WORKSPACE;
        MfmaFwdArgs a = mfma_fwd_shape(B, H, T, D, dtype, causal, w1, w2, kl, kr, flags);
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.lse = lse; a.ut = workspace;
        a.alpha = alpha;
        a.H = H;
        // a dense view goes as dense (strides of extent-1 dimensions may hold anything)
        if (!layout_dense(in_layouts, B, H, T, D)) {
            a.in_sb = in_layouts[0].stride_b; a.in_sh = in_layouts[0].stride_h; a.in_st = in_layouts[0].stride_t;
            if (T == 1) a.in_st = D;  // never used as a step; 0 would read as "dense"
        }
        if (!layout_dense(in_layouts + 3, B, H, T, D)) {
            a.v1_sb = in_layouts[3].stride_b; a.v1_sh = in_layouts[3].stride_h; a.v1_st = in_layouts[3].stride_t;
            if (T == 1) a.v1_st = D;
        }
        // K1, K2 or V2 laid out differently from Q: every tensor on its own layout
        if (!same_layout(in_layouts[0], in_layouts[1]) || !same_layout(in_layouts[0], in_layouts[2]) ||
            !same_layout(in_layouts[0], in_layouts[4])) {
            a.many_views = 1;
            a.at_k1 = tensor_at(in_layouts + 1, H, T, D); a.at_k2 = tensor_at(in_layouts + 2, H, T, D);
            a.at_v2 = tensor_at(in_layouts + 4, H, T, D);
            if (layout_dense(in_layouts, B, H, T, D)) {  // Q itself dense: its strides in (batch, head) terms
                a.in_sb = (long long)H * T * D; a.in_sh = (long long)T * D; a.in_st = D;
            }
        }
        return (int)mfma_tdp_fwd(a, (hipStream_t)stream);
    }
    Views v;
    const void* src[5] = {q, k1, k2, v1, v2};
    rc = plan_all(v, 0, src, in_layouts, 5, workspace ? (char*)workspace + plain : nullptr, B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if ((plain + v.bytes) && (!workspace || workspace_bytes < plain + v.bytes)) return TRITT_ERR_WORKSPACE;
    run_pack(v, B, H, T, D, dtype, (hipStream_t)stream);
    return tritt_tdp_fwd(v.ptr[0], v.ptr[1], v.ptr[2], v.ptr[3], v.ptr[4], o, lse, B, H, T, D, dtype, alpha, causal,
                         k1_window, k2_window, kk_left, kk_right, workspace, plain, flags, stream);
}
// The dot-product-sum kernels on the 16-bit matrix-core path read every strided view where it lies (the packing pass
// and the owner-tile loads take the caller's strides); the fp32 path gets packed copies.
static RowLayout row_layout(const tritt_layout* l, int H, int T, int D) {
    if (!l) return RowLayout{(long long)H * T * D, (long long)T * D, D};
    return RowLayout{l->stride_b, l->stride_h, l->stride_t};
}
static void dps_views(MfmaDpsArgs& a, const tritt_layout* in, const tritt_layout* d_o, int H, int T, int D) {
    a.H = H;
    a.lq = row_layout(in, H, T, D); a.lk1 = row_layout(in ? in + 1 : nullptr, H, T, D);
    a.lk2 = row_layout(in ? in + 2 : nullptr, H, T, D); a.lv1 = row_layout(in ? in + 3 : nullptr, H, T, D);
    a.lv2 = row_layout(in ? in + 4 : nullptr, H, T, D); a.ldo = row_layout(d_o, H, T, D);
}

size_t tritt_dps_fwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags,
                                             const tritt_layout* in_layouts) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_dps(D, dtype, flags)) return round256(tritt_dps_fwd_workspace_bytes(B, H, T, D, dtype, flags));
    Views v;
    const void* none[5] = {};
    if (plan_all(v, 0, none, in_layouts, 5, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    return round256(tritt_dps_fwd_workspace_bytes(B, H, T, D, dtype, flags)) + v.bytes;
}

int tritt_dps_fwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, void* o, float* lse, int B, int H, int T, int D, int dtype,
                          float alpha, int causal, int k_diff, void* workspace, size_t workspace_bytes, unsigned flags,
                          void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o})) return TRITT_ERR_INVALID;
    if (causal && k_diff < 0) return TRITT_ERR_INVALID;
    for (int i = 0; in_layouts && i < 5; ++i)
        if ((rc = check_layout(in_layouts + i, dtype)) != TRITT_OK) return rc;
    const size_t plain = round256(tritt_dps_fwd_workspace_bytes(B, H, T, D, dtype, flags));
    if (use_mfma_dps(D, dtype, flags)) {
        if (!workspace || workspace_bytes < plain) return TRITT_ERR_WORKSPACE;
        MfmaDpsArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o_out = o; a.lse_out = lse; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0; a.k_diff = clampw(k_diff, T);
        a.is_bf16 = dtype == TRITT_BF16;
        dps_views(a, in_layouts, nullptr, H, T, D);
        return (int)mfma_dps_fwd(a, (hipStream_t)stream);
    }
    Views v;
    const void* src[5] = {q, k1, k2, v1, v2};
    rc = plan_all(v, 0, src, in_layouts, 5, workspace ? (char*)workspace + plain : nullptr, B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (!workspace || workspace_bytes < plain + v.bytes) return TRITT_ERR_WORKSPACE;
    run_pack(v, B, H, T, D, dtype, (hipStream_t)stream);
    return tritt_dps_fwd(v.ptr[0], v.ptr[1], v.ptr[2], v.ptr[3], v.ptr[4], o, lse, B, H, T, D, dtype, alpha, causal, k_diff,
                         workspace, plain, flags, stream);
}

size_t tritt_dps_bwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags,
                                             const tritt_layout* in_layouts, const tritt_layout* d_o_layout) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_dps(D, dtype, flags)) return round256(tritt_dps_bwd_workspace_bytes(B, H, T, D, dtype, flags));
    Views v;
    const void* none[5] = {};
    if (plan_all(v, 0, none, in_layouts, 5, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    if (plan_all(v, 5, none, d_o_layout, 1, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    return round256(tritt_dps_bwd_workspace_bytes(B, H, T, D, dtype, flags)) + v.bytes;
}

int tritt_dps_bwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, const void* o, const float* lse, const void* d_o,
                          const tritt_layout* d_o_layout, void* dq, void* dk1, void* dk2, void* dv1, void* dv2, int B,
                          int H, int T, int D, int dtype, float alpha, int causal, int k_diff, void* workspace,
                          size_t workspace_bytes, unsigned flags, void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse, d_o})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o, d_o})) return TRITT_ERR_INVALID;
    if (causal && k_diff < 0) return TRITT_ERR_INVALID;
    for (int i = 0; in_layouts && i < 5; ++i)
        if ((rc = check_layout(in_layouts + i, dtype)) != TRITT_OK) return rc;
    if ((rc = check_layout(d_o_layout, dtype)) != TRITT_OK) return rc;
    const size_t plain = round256(tritt_dps_bwd_workspace_bytes(B, H, T, D, dtype, flags));
    if (use_mfma_dps(D, dtype, flags)) {
        if (any_misaligned({dq, dk1, dk2, dv1, dv2}) || any_null({dq, dk1, dk2, dv1, dv2})) return TRITT_ERR_INVALID;
        if (!workspace || workspace_bytes < plain) return TRITT_ERR_WORKSPACE;
        MfmaDpsArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.d_o = d_o; a.lse_in = lse;
        a.dq = dq; a.dk1 = dk1; a.dk2 = dk2; a.dv1 = dv1; a.dv2 = dv2; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0; a.k_diff = clampw(k_diff, T);
        a.is_bf16 = dtype == TRITT_BF16;
        dps_views(a, in_layouts, d_o_layout, H, T, D);
        return (int)mfma_dps_bwd(a, (hipStream_t)stream);
    }
    Views v;
    const void* src[5] = {q, k1, k2, v1, v2};
    char* tail = workspace ? (char*)workspace + plain : nullptr;
    rc = plan_all(v, 0, src, in_layouts, 5, tail, B, H, T, D, dtype);
    if (rc == TRITT_OK) rc = plan_all(v, 5, &d_o, d_o_layout, 1, tail, B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (!workspace || workspace_bytes < plain + v.bytes) return TRITT_ERR_WORKSPACE;
    run_pack(v, B, H, T, D, dtype, (hipStream_t)stream);
    return tritt_dps_bwd(v.ptr[0], v.ptr[1], v.ptr[2], v.ptr[3], v.ptr[4], o, lse, v.ptr[5], dq, dk1, dk2, dv1, dv2, B, H, T,
                         D, dtype, alpha, causal, k_diff, workspace, plain, flags, stream);
}

// The triple-dot backward on the 16-bit matrix-core path reads the six views where they lie when every row stride
// fits the kernels' 32-bit byte offsets and none is a broadcast along t (the transposing pass reads a pitch of 0 as
// "dense"); otherwise, and on the fp32 path, the views are gathered into the workspace first.
static bool bwd_reads_in_place(const tritt_layout* in, const tritt_layout* d_o, int dtype, int T) {
    auto fits = [&](const tritt_layout* l) {
        return !l || (check_layout(l, dtype) == TRITT_OK && (long long)T * l->stride_t <= 0x7fffffffLL &&
                      (T == 1 || l->stride_t != 0));
    };
    for (int i = 0; in && i < 5; ++i)
        if (!fits(in + i)) return false;
    return fits(d_o);
}

size_t tritt_tdp_bwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, int causal, int k1_window,
                                             int k2_window, int kk_left, int kk_right, unsigned flags,
                                             const tritt_layout* in_layouts, const tritt_layout* d_o_layout) {
    if (check_common(B, H, T, D, dtype) != TRITT_OK) return 0;
    if (use_mfma_bwd(T, D, dtype, causal, clampw(k1_window, T), clampw(k2_window, T), clampw(kk_left, T), clampw(kk_right, T),
                     flags) &&
        bwd_reads_in_place(in_layouts, d_o_layout, dtype, T))
        return round256(tritt_tdp_bwd_workspace_bytes(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags));
    Views v;
    const void* none[5] = {};
    if (plan_all(v, 0, none, in_layouts, 5, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    if (plan_all(v, 5, none, d_o_layout, 1, nullptr, B, H, T, D, dtype) != TRITT_OK) return 0;
    return round256(tritt_tdp_bwd_workspace_bytes(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags)) +
           v.bytes;
}

int tritt_tdp_bwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, const void* o, const float* lse, const void* d_o,
                          const tritt_layout* d_o_layout, void* dq, void* dk1, void* dk2, void* dv1, void* dv2, int B,
                          int H, int T, int D, int dtype, float alpha, int causal, int k1_window, int k2_window,
                          int kk_left, int kk_right, void* workspace, size_t workspace_bytes, unsigned flags,
                          void* stream) {
    if (empty_problem(B, H, T)) return check_common(1, 1, 1, D, dtype);
    int rc = check_common(B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (any_null({q, k1, k2, v1, v2, o, lse, d_o})) return TRITT_ERR_INVALID;
    if (any_misaligned({q, k1, k2, v1, v2, o, d_o})) return TRITT_ERR_INVALID;
    if (!dq && !dk1 && !dk2 && !dv1 && !dv2) return TRITT_OK;
    if (causal && (k1_window < 0 || k2_window < 0 || kk_left < 0 || kk_right < 0)) return TRITT_ERR_INVALID;
    for (int i = 0; in_layouts && i < 5; ++i)
        if ((rc = check_layout(in_layouts + i, dtype)) != TRITT_OK) return rc;
    if ((rc = check_layout(d_o_layout, dtype)) != TRITT_OK) return rc;
    const size_t plain =
        round256(tritt_tdp_bwd_workspace_bytes(B, H, T, D, dtype, causal, k1_window, k2_window, kk_left, kk_right, flags));
    const int w1 = clampw(k1_window, T), w2 = clampw(k2_window, T), kl = clampw(kk_left, T), kr = clampw(kk_right, T);
    if (use_mfma_bwd(T, D, dtype, causal, w1, w2, kl, kr, flags) && (in_layouts || d_o_layout) &&
        bwd_reads_in_place(in_layouts, d_o_layout, dtype, T)) {
        if (any_misaligned({dq, dk1, dk2, dv1, dv2})) return TRITT_ERR_INVALID;
        if ((flags & TRITT_FLAG_SPLIT_OPERANDS) && !use_split(D, dtype, flags)) return TRITT_ERR_UNSUPPORTED;
        if (!workspace || workspace_bytes < plain) return TRITT_ERR_WORKSPACE;
        MfmaBwdArgs a{};
        a.q = q; a.k1 = k1; a.k2 = k2; a.v1 = v1; a.v2 = v2; a.o = o; a.d_o = d_o; a.lse = lse;
        a.dq = dq; a.dk1 = dk1; a.dk2 = dk2; a.dv1 = dv1; a.dv2 = dv2; a.workspace = workspace;
        a.BH = B * H; a.T = T; a.D = D; a.alpha = alpha; a.causal = causal ? 1 : 0;
        a.is_bf16 = dtype == TRITT_BF16;
        a.windowed = full_windows(T, causal, w1, w2, kl, kr) ? 0 : 1;
        a.k1_window = w1; a.k2_window = w2; a.kk_left = kl; a.kk_right = kr;
        a.deterministic = (flags & TRITT_FLAG_FLOAT_ATOMICS) ? 0 : 1;
        a.split = use_split(D, dtype, flags) ? 1 : 0;
        a.H = H;
        a.at_q = tensor_at(in_layouts, H, T, D); a.at_k1 = tensor_at(in_layouts ? in_layouts + 1 : nullptr, H, T, D);
        a.at_k2 = tensor_at(in_layouts ? in_layouts + 2 : nullptr, H, T, D);
        a.at_v1 = tensor_at(in_layouts ? in_layouts + 3 : nullptr, H, T, D);
        a.at_v2 = tensor_at(in_layouts ? in_layouts + 4 : nullptr, H, T, D);
        a.at_do = tensor_at(d_o_layout, H, T, D);
        return (int)mfma_tdp_bwd(a, (hipStream_t)stream);
    }
    Views v;
    const void* src[5] = {q, k1, k2, v1, v2};
    char* tail = workspace ? (char*)workspace + plain : nullptr;
    rc = plan_all(v, 0, src, in_layouts, 5, tail, B, H, T, D, dtype);
    if (rc == TRITT_OK) rc = plan_all(v, 5, &d_o, d_o_layout, 1, tail, B, H, T, D, dtype);
    if (rc != TRITT_OK) return rc;
    if (!workspace || workspace_bytes < plain + v.bytes) return TRITT_ERR_WORKSPACE;
    run_pack(v, B, H, T, D, dtype, (hipStream_t)stream);
    return tritt_tdp_bwd(v.ptr[0], v.ptr[1], v.ptr[2], v.ptr[3], v.ptr[4], o, lse, v.ptr[5], dq, dk1, dk2, dv1, dv2, B, H, T,
                         D, dtype, alpha, causal, k1_window, k2_window, kk_left, kk_right, workspace, plain, flags, stream);
}

}  // extern "C"
