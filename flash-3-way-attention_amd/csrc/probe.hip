// Calibration kernel behind tritt_probe_mfma: what the matrix pipes of this chip sustain when they do nothing
// but bf16 MFMAs.  A benchmark divides the result by the published peak to learn the clock the chip holds under
// a matrix load (the peak assumes the nominal clock).
#include "../../include/trittention_hip.h"

#include "mfma.hpp"

namespace tritt {

// Every wave issues `iters` rounds of four independent 32x32x16 bf16 MFMAs (four accumulators, so no MFMA waits
// for the one before it); eight waves per workgroup, two per SIMD.
__global__ __launch_bounds__(512) void mfma_probe_kernel(float* __restrict__ out, int iters) {
    using M = Mma<__bf16>;
    M::v8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (__bf16)(0.001f * (float)((threadIdx.x + e) & 7));
        b[e] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + e) & 7));
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0.f;
    for (int it = 0; it < iters; ++it) {
        c0 = M::mma(a, b, c0);
        c1 = M::mma(a, b, c1);
        c2 = M::mma(a, b, c2);
        c3 = M::mma(a, b, c3);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace tritt

extern "C" int tritt_probe_mfma(float* out, int blocks, int iters, void* stream) {
    if (!out || blocks <= 0 || iters <= 0) return TRITT_ERR_INVALID;
    hipLaunchKernelGGL(tritt::mfma_probe_kernel, dim3(blocks), dim3(512), 0, (hipStream_t)stream, out, iters);
    return (int)hipGetLastError();
}
