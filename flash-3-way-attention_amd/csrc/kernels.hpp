// Internal launch interfaces between capi.hip and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace tritt {

// Tuning overrides (tritt_set_tuning; initial values from the environment, read once per process, so that a
// workspace query and the launch that follows it agree).  0 = automatic.
struct Knobs {
    int fwd_splits;      // TRITT_TUNE_FWD_SPLITS / env TRITT_FWD_SPLITS: workgroups per query tile, forward (1..8)
    int fwd_band;        // TRITT_TUNE_FWD_BAND / env TRITT_FWD_BAND: -1 switches the band-resident forward off
    int bwd_splits;      // TRITT_TUNE_BWD_SPLITS / env TRITT_BWD_SPLITS: workgroups per query tile, backward (1..16)
    int bwd128_variant;  // TRITT_TUNE_BWD128_WAVES / env TRITT_BWD128_VARIANT=w8|w4: the 32-query kernels (default: 16 queries per wave)
    int f32_valu;        // TRITT_TUNE_F32_VALU: 1 = fp32 tensors take the VALU kernels at every head dimension
    int dps_waves;       // TRITT_TUNE_DPS_WAVES: waves per workgroup of the dot-product-sum MFMA kernels at D = 64 (2 | 4)
    int dps_pair;        // TRITT_TUNE_DPS_PAIR: 1 / -1 = owner tiles always / never paired in those kernels
    int dps_shared;      // TRITT_TUNE_DPS_SHARED: 1 / -1 = the shared-tile dot-product-sum kernels always / never
};
Knobs knobs();

// Where slice (b, h) of a [B,H,T,D] tensor starts and how far its rows lie apart, in elements (a strided view of the
// caller's, or a dense tensor: sb = H T D, sh = T D, st = D).
struct TensorAt {
    long long sb, sh;
    unsigned st;
};
inline TensorAt dense_at(int H, int T, int D) { return TensorAt{(long long)H * T * D, (long long)T * D, (unsigned)D}; }

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per (device, kernel): the attribute belongs to the
// device's copy of the kernel, and a process may drive several devices.
hipError_t ensure_dynamic_smem(const void* kernel, size_t bytes);

// fp32 [BH, T, D] operands of the VALU triple-dot kernels (u = SiLU(V1)).
struct GenericTdpArgs {
    const float *q, *k1, *k2, *u, *v2;
    float* o;            // forward output
    float* lse;          // forward output [BH, T]
    const float* lse_in; // backward input
    const float* d_o;    // backward input
    const float* delta;  // backward input [BH, T] = rowsum(dO * O)
    float *dq, *dk1, *dk2, *du, *dv2;
    int BH, T, D;
    float alpha;
    int causal, k1_window, k2_window, kk_left, kk_right;
};
hipError_t generic_tdp_fwd(const GenericTdpArgs& a, hipStream_t st);
hipError_t generic_tdp_bwd(const GenericTdpArgs& a, hipStream_t st);

// fp32 MFMA triple-dot kernels (D = 32 or 64, any mask): same operands as the VALU kernels
bool f32_mfma_tdp_supported(int D);
hipError_t f32_mfma_tdp_fwd(const GenericTdpArgs& a, hipStream_t st);
// backward: `scratch` = f32_mfma_tdp_bwd_scratch_elems() 64-bit words (fixed-point accumulators of the four
// key / value gradients; zeroed by the call)
size_t f32_mfma_tdp_bwd_scratch_elems(int BH, int T, int D);
hipError_t f32_mfma_tdp_bwd(const GenericTdpArgs& a, long long* scratch, hipStream_t st);

// The first `tiles` query tiles (32 queries each) of a 16-bit triple-dot backward, computed in fp32 from the
// 16-bit tensors (D = 32, 64 or 128) and added to the accumulators of the 16-bit MFMA backward, which then starts
// at the tile after them.
struct FirstTileArgs {
    const void *q, *d_o, *k1, *u, *k2, *v2;  // 16-bit; u = SiLU(V1) is dense [BH][T][D]
    // the other five lie where the caller has them: H heads per batch entry and these strides (H = 0: all dense)
    int H;
    TensorAt at_q, at_do, at_k1, at_k2, at_v2;
    // scratch, [BH][T] floats each: the covered rows' LSE and Delta, recomputed in fp32 (tiles == 1: delta_f32 holds
    // the per-round partials of tile 0 instead, [BH][32][4][3])
    float *lse_f32, *delta_f32;
    void* dq0_acc;                            // tiles == 1 and acc_q null: [BH][32][D] accumulator of the tile's dQ / alpha
    void* dq;                                 // written when acc_q is null
    void *acc_k2, *acc_v2, *acc_k1, *acc_u;   // fixed point (long long) or float
    void* acc_q;                              // dQ / alpha accumulator of a split backward, or null
    // fixed-point accumulators (common.hpp): the slices' scale partials, the rows' poison words and the bias of the
    // scale; scale_parts null: float accumulators
    const unsigned* scale_parts;
    unsigned* poison;
    int scale_bias;
    int BH, T, D, is_bf16;
    float alpha;
    int causal, k1_window, k2_window, kk_left, kk_right;
    bool want_q, want_k2, want_k1;
    int tiles;
    int round_parts;  // tiles > 1: workgroups per query tile (its rounds of eight rows dealt out); above 1 needs acc_q when dQ is wanted
};
hipError_t f32_mfma_tdp_bwd_first_tile(const FirstTileArgs& a, hipStream_t st);
// Workgroups per query tile of the fp32 matrix-core backward over all tiles: one workgroup walks a tile's rounds (of
// eight rows) one after another, so a grid that leaves most compute units idle (short sequences, few heads) is
// dealt out by rounds as well.
int f32_round_parts(int BH, int T);

// fp32 operands of the dot-product-sum kernels (two chained attention passes).
struct DpsArgs {
    const float *q, *k1, *k2, *u, *v2;
    float* o;
    float* lse;          // forward output / backward input (natural log) [BH, T]
    const float* d_o;
    const float* o_in;
    float *dq, *dk1, *dk2, *du, *dv2;
    // scratch, all fp32: r, w, dw, dr, dk2_part [BH,T,D]; lse1, delta, dlse1, delta1 [BH,T]
    float *r, *w, *dw, *dr, *dk2_part, *lse1, *delta, *dlse1, *delta1;
    int BH, T, D;
    float alpha;
    int causal, k_diff;
};
hipError_t dps_fwd(const DpsArgs& a, hipStream_t st);
hipError_t dps_bwd(const DpsArgs& a, hipStream_t st);
// the same two calls with the attention kernels on the fp32 matrix cores (D = 32 or 64)
bool f32_mfma_dps_supported(int D);
hipError_t f32_mfma_dps_fwd(const DpsArgs& a, hipStream_t st);
hipError_t f32_mfma_dps_bwd(const DpsArgs& a, hipStream_t st);

// 16-bit MFMA triple-dot forward (any mask; D = 32, 64 or 128).
struct MfmaFwdArgs {
    const void *q, *k1, *k2, *v1, *v2;
    void* o;
    float* lse;
    void* ut;  // scratch: mfma_tdp_fwd_workspace() bytes
    int BH, T, D;
    float alpha;
    int causal;
    int is_bf16;  // else fp16
    int windowed;  // some window can exclude a pair with j, k <= q: the banded instantiation
    int k1_window, k2_window, kk_left, kk_right;
    // split operands (D = 32, 64): the Q (.) K2 operand of the score products as a hi + lo pair of 16-bit numbers;
    // `o` then holds two [BH][T][D] tensors, the output and its rounding residual
    int split;
    // Strided inputs: element (b, h, t, d) of Q, K1, K2 and V2 at b in_sb + h in_sh + t in_st + d elements, of V1 at the
    // v1_* strides; H = heads (BH = batch * H).  in_st == 0 / v1_st == 0: dense [BH][T][D].  Row strides below 2^32.
    long long in_sb, in_sh, in_st, v1_sb, v1_sh, v1_st;
    int H;
    // many_views != 0: K1, K2 and V2 lie on layouts of their own (at_k1, at_k2, at_v2; in_* is then Q's alone)
    int many_views;
    TensorAt at_k1, at_k2, at_v2;
};
bool mfma_tdp_split_supported(int D, int dtype_is_16bit);
// needs BH, T, D, causal, windowed, split and the four windows of `a`
size_t mfma_tdp_fwd_workspace(const MfmaFwdArgs& a);
bool mfma_tdp_fwd_supported(int D, int dtype_is_16bit);
hipError_t mfma_tdp_fwd(const MfmaFwdArgs& a, hipStream_t st);

// 16-bit MFMA triple-dot backward (any mask; D = 32, 64 or 128).
struct MfmaBwdArgs {
    const void *q, *k1, *k2, *v1, *v2, *o, *d_o;
    // H > 0: q, k1, k2, v1, v2 and d_o are strided views (heads per batch entry, strides in elements) that the kernels
    // read where they lie; H == 0: all dense [BH][T][D]
    int H;
    TensorAt at_q, at_k1, at_k2, at_v1, at_v2, at_do;
    const float* lse;
    void *dq, *dk1, *dk2, *dv1, *dv2;
    void* workspace;  // mfma_tdp_bwd_workspace() bytes
    int BH, T, D;
    float alpha;
    int causal;
    int is_bf16;
    int windowed;  // some window can exclude a pair with j, k <= q: the banded kernels
    int k1_window, k2_window, kk_left, kk_right;
    int deterministic;  // 64-bit fixed-point accumulators: bitwise reproducible gradients
    // split operands (D = 32, 64): Q (.) K2 and dO (.) V2 as hi + lo pairs; `o` holds the output followed by its
    // rounding residual (what the forward wrote under the same flag), and Delta is formed from their sum
    int split;
};
size_t mfma_tdp_bwd_workspace(int BH, int T, int D, bool deterministic);
bool mfma_tdp_bwd_supported(int D, int dtype_is_16bit);
hipError_t mfma_tdp_bwd(const MfmaBwdArgs& a, hipStream_t st);

// 16-bit MFMA dot-product-sum (two chained banded attentions; D = 32, 64 or 128).
// strides of a [B,H,T,D] view in elements (tritt_layout)
struct RowLayout {
    long long sb, sh, st;
};
struct MfmaDpsArgs {
    const void *q, *k1, *k2, *v1, *v2;
    // H > 0: q, k1, k2, v1, v2 and d_o are views with these strides (read where they lie); H == 0: all dense
    int H;
    RowLayout lq, lk1, lk2, lv1, lv2, ldo;
    void* o_out;          // forward output
    float* lse_out;       // forward output [BH, T] (natural log)
    const void *o, *d_o;  // backward inputs
    const float* lse_in;  // backward input
    void *dq, *dk1, *dk2, *dv1, *dv2;
    void* workspace;      // mfma_dps_{fwd,bwd}_workspace() bytes
    int BH, T, D;
    float alpha;
    int causal, k_diff;
    int is_bf16;
};
size_t mfma_dps_fwd_workspace(int BH, int T, int D);
size_t mfma_dps_bwd_workspace(int BH, int T, int D);
bool mfma_dps_supported(int D, int dtype_is_16bit);
hipError_t mfma_dps_fwd(const MfmaDpsArgs& a, hipStream_t st);
hipError_t mfma_dps_bwd(const MfmaDpsArgs& a, hipStream_t st);

}  // namespace tritt
