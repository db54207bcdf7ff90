// MFMA (gfx950) wrappers shared by the 16-bit kernels: 32x32x16 tiles, wave64.
//
// v_mfma_f32_32x32x16_{bf16,f16}: D[32x32] = A[32x16] * B[16x32] + C.
//   A operand: lane l holds A[row = l%32][k = 8*(l/32) .. +8]
//   B operand: lane l holds B[k = 8*(l/32) .. +8][col = l%32]
//   C/D:       lane l holds D[row = 8*(i/4) + 4*(l/32) + i%4][col = l%32], i = 0..15
#pragma once
#include "common.hpp"

namespace tritt {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) float f32x2;

template <typename E>
struct Mma;

template <>
struct Mma<__bf16> {
    using v8 = bf16x8;
    using v2 = bf16x2;
    static __device__ __forceinline__ f32x16 mma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ v2 pack(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_convertvector(v, v2);
    }
    // c + p.x + p.y
    static __device__ __forceinline__ float add_pair(v2 p, float c) {
        const v2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(p, ones, c, false);
    }
};

template <>
struct Mma<_Float16> {
    using v8 = f16x8;
    using v2 = f16x2;
    static __device__ __forceinline__ f32x16 mma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ v2 pack(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_convertvector(v, v2);
    }
    static __device__ __forceinline__ float add_pair(v2 p, float c) {
        const v2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(p, ones, c, false);
    }
};

// row of the 32x32 C/D tile held in register i of a lane in half g = lane/32
__device__ __forceinline__ constexpr int c_row(int g, int i) { return 8 * (i / 4) + 4 * g + (i % 4); }

// The score tiles are computed transposed (rows = key index j, cols = virtual query row) and the
// K1 rows fed to the MFMA are permuted so that register i of lane-half g holds key
//   j = 16*(i/8) + 8*g + i%8
// i.e. registers 0..7 / 8..15 of a lane are exactly the 8 consecutive k-slots that lane must
// supply as the A operand of the following P*U product: no cross-lane movement between the two.
__device__ __forceinline__ constexpr int key_of(int g, int i) { return 16 * (i / 8) + 8 * g + (i % 8); }
// inverse: which key offset must sit in MFMA row r of the K1 operand
__device__ __forceinline__ int key_of_row(int r) {
    const int g = (r >> 2) & 1, i = ((r >> 3) << 2) | (r & 3);
    return key_of(g, i);
}

}  // namespace tritt
