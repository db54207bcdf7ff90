/* trittention_hip.h — C ABI of libtrittention_hip.so (MI355X / gfx950).
 *
 * The library implements the "trittention" (3-way attention) hot path of
 * flash-3-way-attention with hand-written HIP kernels.  Every entry point
 * takes plain device pointers, sizes and a HIP stream; no framework types
 * cross this boundary.  All tensors are contiguous row-major [B, H, T, D].
 * `lse` is [B, H, T] fp32 (natural-log logsumexp of the scaled, masked
 * scores of each query row).
 *
 * Each function names the reference interface it replaces (paths relative
 * to the reference repository's src/flash_trittention/).
 *
 * Return value: 0 on success; a negative TRITT_ERR_* code when the
 * arguments are rejected before anything is launched; a positive value is
 * the hipError_t reported by the launch.  Nothing is allocated or freed by
 * these calls: scratch memory is passed in by the caller (`workspace`), its
 * required size is returned by the matching *_workspace_bytes function.
 * Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 * null stream) and the calls do not synchronise.  A problem with B, H or T
 * equal to 0 is a successful no-op: nothing is launched, no pointer is read
 * (they may be NULL) and its workspace size is 0.
 */
#ifndef TRITTENTION_HIP_H
#define TRITTENTION_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of q,k1,k2,v1,v2,o,dO and of the five gradients */
enum { TRITT_F32 = 0, TRITT_BF16 = 1, TRITT_F16 = 2 };

enum {
    TRITT_OK = 0,
    TRITT_ERR_INVALID = -1,     /* null or misaligned pointer, negative size, bad dtype,
                                   B*H above 65535 or B*H*T above 2^31-1                    */
    TRITT_ERR_HEAD_DIM = -2,    /* D not one of 8, 16, 32, 64, 128                         */
    TRITT_ERR_WORKSPACE = -3,   /* workspace missing or smaller than *_workspace_bytes     */
    TRITT_ERR_UNSUPPORTED = -4, /* requested implementation cannot run this configuration */
    TRITT_ERR_SCRATCH_LIMIT = -5 /* tritt_tdp_fwd_static_scratch: the problem needs more scratch
                                    than TRITT_STATIC_SCRATCH_BYTES                         */
};

/* `flags` bits */
enum {
    TRITT_FLAG_AUTO = 0,
    TRITT_FLAG_FORCE_GENERIC = 1, /* use the fp32 VALU kernels even where an MFMA kernel exists */
    TRITT_FLAG_FORCE_MFMA = 2,    /* fail with TRITT_ERR_UNSUPPORTED instead of falling back    */
    TRITT_FLAG_FLOAT_ATOMICS = 4, /* tritt_tdp_bwd, MFMA path: accumulate the shared gradients with fp32
                                     atomics instead of 64-bit fixed point (see tritt_tdp_bwd)     */
    TRITT_FLAG_SPLIT_OPERANDS = 8 /* tritt_tdp_fwd / tritt_tdp_bwd, 16-bit tensors, D = 32 or 64: what the
                                     reference's convert_to_float32=True asks of its kernels
                                     (triple_dot_product/flash_trittention.py:408, kernels/bwd_dq.py:197,219),
                                     at matrix-core speed.  The operands Q (.) K2 and dO (.) V2 of the score
                                     products are kept to 16 mantissa bits (a hi + lo pair of 16-bit numbers,
                                     two MFMAs per k-step), so scores and dP carry fp32 accumulation error only.
                                     `o` then points to TWO consecutive [B,H,T,D] tensors: the output, and the
                                     rounding residual of every output element (fp32 value minus stored value;
                                     written by tritt_tdp_fwd, read by tritt_tdp_bwd for Delta = rowsum(dO * O)).
                                     Other configurations: TRITT_ERR_UNSUPPORTED (use TRITT_FLAG_FORCE_GENERIC,
                                     the fp32 kernels, there).                                          */
};

/* Library version (major*10000 + minor*100 + patch) and a static, human
 * readable description of a return code. */
int tritt_version(void);
const char* tritt_status_string(int status);

/* Tuning overrides for sweeps and tests; production callers never need them.  Each knob
 * starts from an environment variable that is read once per process (the first time any
 * entry point needs it), so a *_workspace_bytes query and the launch that follows always see
 * the same value; tritt_set_tuning changes a knob afterwards, stores its previous value in
 * *previous (which may be NULL) and returns TRITT_OK, or TRITT_ERR_INVALID for an unknown knob.
 * 0 = automatic.  Process-wide: do not change a knob while another thread is inside the library.
 *   TRITT_TUNE_FWD_SPLITS   (env TRITT_FWD_SPLITS)     workgroups per query tile in the triple-dot forward, 1..8
 *   TRITT_TUNE_FWD_BAND     (env TRITT_FWD_BAND=0)     -1: narrow windowed masks take the streaming forward
 *                                                      instead of the band-resident one
 *   TRITT_TUNE_BWD_SPLITS   (env TRITT_BWD_SPLITS)     workgroups per query tile in the triple-dot backward, 1..16
 *   TRITT_TUNE_BWD128_WAVES (env TRITT_BWD128_VARIANT=w8|w4)  the D = 128 backward under full windows: 0 = 16 queries per
 *                           wave on 16x16x32 tiles (the default); 8 | 4 = the 32-query kernels with 8 or 4 waves
 *   TRITT_TUNE_F32_VALU     (env TRITT_F32_VALU=1)     1: the fp32 path runs the VALU kernels at every head dimension (instead of the
 *                           fp32 MFMA kernels at D = 32, 64 and 128)
 *   TRITT_TUNE_DPS_WAVES    waves per workgroup of the dot-product-sum MFMA kernels at D = 64: 2 | 4
 *   TRITT_TUNE_DPS_PAIR     dot-product-sum MFMA kernels: 1 = a workgroup always takes two owner tiles (a long and a
 *                           short one), -1 = never
 *   TRITT_TUNE_DPS_SHARED   dot-product-sum on the 16-bit matrix cores: 1 = always the kernels whose workgroups own 128 rows
 *                           and share the streamed tiles through LDS, -1 = never (0: the forward passes from 1024 such
 *                           workgroups on, the backward kernels at D = 64 and 128 from 512 on) */
enum { TRITT_TUNE_FWD_SPLITS = 0, TRITT_TUNE_FWD_BAND = 1, TRITT_TUNE_BWD_SPLITS = 2, TRITT_TUNE_BWD128_WAVES = 3,
       TRITT_TUNE_F32_VALU = 4, TRITT_TUNE_DPS_WAVES = 5, TRITT_TUNE_DPS_PAIR = 6, TRITT_TUNE_DPS_SHARED = 7,
       TRITT_TUNE_COUNT_ = 8 };
int tritt_set_tuning(int knob, int value, int* previous);

/* ---- triple-dot-product:  s[q,j,k] = alpha * sum_d Q[q,d] K1[j,d] K2[k,d] ----------------
 * O[q] = sum_{j,k} softmax_{(j,k)}(s[q]) * SiLU(V1[j]) * V2[k].
 * causal != 0 masks (reference triple_dot_product/trittention_pytorch.py:68-75)
 *   j>q | k>q | q>j+k1_window | q>k+k2_window | j+kk_left<k | k+kk_right<j ;
 * pass T (or more) for a window to disable it.  causal == 0: no mask, windows ignored.
 *
 * tritt_tdp_fwd replaces FlashTrittention.forward + the _tritt_fwd launch
 *   (triple_dot_product/flash_trittention.py:16-139, kernels/fwd.py:9-225): it also
 *   applies SiLU to V1 itself and writes the final lse (the reference's M + log L).
 * tritt_tdp_bwd replaces FlashTrittention.backward and its five launches
 *   (triple_dot_product/flash_trittention.py:141-393, kernels/bwd_{dq,dk1,dk2,dv1,dv2}.py),
 *   including Delta = rowsum(dO*O) and the SiLU' factor on dV1.  Any of dq, dk1, dk2, dv1, dv2 may
 *   be NULL: that gradient is not wanted, and a kernel launch that only serves unwanted gradients
 *   is skipped (the launches produce {dq, dk2, dv2} and {dk1, dv1}; the fp32 kernels {dq},
 *   {dk2, dv2} and {dk1, dv1}).  On the 16-bit MFMA path
 *   (16-bit tensors, D = 32, 64 or 128, any mask) the workgroups of different query tiles add their
 *   shares of dK1/dV1/dK2/dV2 (and of dQ, when a small grid splits a tile's rows) to common
 *   accumulators.  The shares are added as 64-bit fixed point with integer atomics, whose result
 *   does not depend on the order of arrival: like the reference's owner-computes kernels, and
 *   like every other entry point here, the call is bitwise reproducible from run to run
 *   (measured cost against fp32 atomics: none).  The fixed-point scale is a power of two chosen
 *   per (batch, head) slice from the largest finite |dO| of the slice: steps of 2^-30 of that
 *   magnitude (2^-36 on the fp32 matrix-core kernels), sums up to 2^33 (2^27) times it, so the
 *   backward is exactly homogeneous in dO for powers of two (loss scaling, mean-reduced losses)
 *   and has no absolute floor, like the reference's fp32 accumulators
 *   (triple_dot_product/kernels/bwd_dk1.py:239-258).  A share that is NaN, Inf or beyond the
 *   accumulator's range makes that row of that gradient NaN in the output.
 *   TRITT_FLAG_FLOAT_ATOMICS selects fp32 atomics instead (reproducible to rounding only;
 *   accumulators half the size: pass the same flags to tritt_tdp_bwd_workspace_bytes).  Workspace of the MFMA path: about 15 (fixed point: 25) times
 *   one 16-bit [B,H,T,D] tensor (five accumulators, four transposed copies, SiLU(V1)).
 */
size_t tritt_tdp_fwd_workspace_bytes(int B, int H, int T, int D, int dtype, int causal,
                                     int k1_window, int k2_window, int kk_left, int kk_right,
                                     unsigned flags);
int tritt_tdp_fwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                  void* o, float* lse,
                  int B, int H, int T, int D, int dtype, float alpha, int causal,
                  int k1_window, int k2_window, int kk_left, int kk_right,
                  void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/* tritt_tdp_fwd_static_scratch has no counterpart in the reference.  It is tritt_tdp_fwd for
 * callers that cannot allocate device memory at all (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the scratch that tritt_tdp_fwd takes as
 * `workspace` lives in a static device array inside the library instead, of
 * TRITT_STATIC_SCRATCH_BYTES bytes per GPU, held until the process ends.  The call allocates
 * and frees nothing.  Problems whose tritt_tdp_fwd_workspace_bytes() exceeds that size are
 * rejected with TRITT_ERR_SCRATCH_LIMIT before anything is launched (32 MiB covers the
 * forward up to B*H*T*D = 16 Mi 16-bit elements, e.g. B=1 H=16 T=4096 D=128).  All calls on
 * one GPU share the one array: calls that overlap in time on the same GPU (different
 * streams or threads) race; serialise them.  Results are identical to tritt_tdp_fwd's.
 * tritt_static_scratch_bytes() returns the limit the library was built with. */
#define TRITT_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
size_t tritt_static_scratch_bytes(void);
int tritt_tdp_fwd_static_scratch(const void* q, const void* k1, const void* k2, const void* v1,
                                 const void* v2, void* o, float* lse,
                                 int B, int H, int T, int D, int dtype, float alpha, int causal,
                                 int k1_window, int k2_window, int kk_left, int kk_right,
                                 unsigned flags, void* stream);

size_t tritt_tdp_bwd_workspace_bytes(int B, int H, int T, int D, int dtype, int causal,
                                     int k1_window, int k2_window, int kk_left, int kk_right,
                                     unsigned flags);
int tritt_tdp_bwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                  const void* o, const float* lse, const void* d_o,
                  void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                  int B, int H, int T, int D, int dtype, float alpha, int causal,
                  int k1_window, int k2_window, int kk_left, int kk_right,
                  void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/* ---- dot-product-sum:  s[q,s,t] = alpha * (K2[t].Q[q] + K1[s].K2[t]) ---------------------
 * O[q] = sum_{s,t} softmax_{(s,t)}(s[q]) * SiLU(V1[s]) * V2[t].
 * causal != 0 keeps s <= t <= q and t - s <= k_diff
 *   (reference dot_product_sum/trittention_pytorch.py:47-51); causal == 0: no mask.
 *
 * tritt_dps_fwd replaces TrittentionTritonFunction.forward + _tritt_fwd
 *   (dot_product_sum/trittention_triton.py:17-125, kernels/fwd_kernel.py:225-375);
 *   `lse` is the tensor that function returns as `m`.
 * tritt_dps_bwd replaces TrittentionTritonFunction.backward with
 *   _tritt_bwd_preprocess, _tritt_bwd_dq and _tritt_bwd_dk_dv
 *   (dot_product_sum/trittention_triton.py:127-359, kernels/bwd_preprocess.py:6,
 *   kernels/bwd_dq_kernel.py:30, kernels/bwd_dk1_dv1_kernel.py:31).  It uses no atomics:
 *   results are bitwise reproducible from run to run.
 */
size_t tritt_dps_fwd_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags);
int tritt_dps_fwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                  void* o, float* lse,
                  int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                  void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

size_t tritt_dps_bwd_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags);
int tritt_dps_bwd(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                  const void* o, const float* lse, const void* d_o,
                  void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                  int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                  void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/* ---- strided inputs ------------------------------------------------------------------------
 * The entry points above take dense [B,H,T,D] tensors.  The reference accepts views of any strides and copies them
 * (triple_dot_product/flash_trittention.py:64-68,153; dot_product_sum/trittention_triton.py:43-47;
 * tests/test_dot_product_sum.py:121-134); a projection layer usually hands over [B,T,H,D] (or a slice of a fused
 * [B,T,5,H,D]) transposed.  The *_strided entry points take such views as they are: a tritt_layout gives the
 * element strides of a view whose last dimension is dense (element (b,h,t,d) at
 * ptr + b*stride_b + h*stride_h + t*stride_t + d).  `in_layouts` points to five of them, for q, k1, k2, v1, v2 in this
 * order (NULL: all dense); `d_o_layout` to the one of dO (NULL: dense).  Strides are non-negative multiples of 16
 * bytes (8 elements of a 16-bit type, 4 of fp32), the row stride below 2^31 elements, pointers 16-byte aligned as
 * before; else TRITT_ERR_INVALID.  Outputs (o, lse, the gradients) and the saved `o` are dense.
 * On the 16-bit matrix-core paths the views are read where they lie, and the workspace is the dense call's:
 *   tritt_tdp_fwd_strided: V1 through the SiLU/transpose pass it makes anyway, Q, K1, K2 and V2 inside the main kernel
 *     (one instantiation for four tensors on a common layout: slices of one fused tensor, or tensors transposed alike;
 *     another for a layout per tensor);
 *   tritt_tdp_bwd_strided: all six views, each on its own layout (the transposing pass, the row kernels, the fp32
 *     kernels of the first query tile and the final pass take the strides);
 *   tritt_dps_fwd_strided, tritt_dps_bwd_strided: all views, each on its own layout (the packing pass, the owner-tile
 *     loads and the epilogues take the strides; broadcast views with a stride of zero included).
 *   The triple-dot calls read in place only while T * stride_t stays below 2^31 elements and no view is a broadcast
 *   along t.
 * Everywhere else (fp32 tensors, head dimensions without a matrix-core kernel, the two triple-dot limits just named)
 *   the views that are not dense are first gathered into the tail of the workspace by one launch for
 *   all of them, and the dense code runs on the copies: one read and one write of each such tensor, no allocation,
 *   no per-tensor launches.
 * The *_strided_workspace_bytes queries take the same layouts and return the dense call's size plus the room of such
 * copies where they are made; everything else is as in the dense call of the same name. */
typedef struct tritt_layout {
    long long stride_b, stride_h, stride_t;
} tritt_layout;

size_t tritt_tdp_fwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, int causal,
                                             int k1_window, int k2_window, int kk_left, int kk_right,
                                             unsigned flags, const tritt_layout* in_layouts);
int tritt_tdp_fwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, void* o, float* lse,
                          int B, int H, int T, int D, int dtype, float alpha, int causal,
                          int k1_window, int k2_window, int kk_left, int kk_right,
                          void* workspace, size_t workspace_bytes, unsigned flags, void* stream);
size_t tritt_tdp_bwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, int causal,
                                             int k1_window, int k2_window, int kk_left, int kk_right,
                                             unsigned flags, const tritt_layout* in_layouts,
                                             const tritt_layout* d_o_layout);
int tritt_tdp_bwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, const void* o, const float* lse,
                          const void* d_o, const tritt_layout* d_o_layout,
                          void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                          int B, int H, int T, int D, int dtype, float alpha, int causal,
                          int k1_window, int k2_window, int kk_left, int kk_right,
                          void* workspace, size_t workspace_bytes, unsigned flags, void* stream);
size_t tritt_dps_fwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags,
                                             const tritt_layout* in_layouts);
int tritt_dps_fwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, void* o, float* lse,
                          int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                          void* workspace, size_t workspace_bytes, unsigned flags, void* stream);
size_t tritt_dps_bwd_strided_workspace_bytes(int B, int H, int T, int D, int dtype, unsigned flags,
                                             const tritt_layout* in_layouts, const tritt_layout* d_o_layout);
int tritt_dps_bwd_strided(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                          const tritt_layout* in_layouts, const void* o, const float* lse,
                          const void* d_o, const tritt_layout* d_o_layout,
                          void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                          int B, int H, int T, int D, int dtype, float alpha, int causal, int k_diff,
                          void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/* Calibration for benchmarks (no counterpart in the reference).  Launches `blocks` workgroups of
 * eight waves that each issue iters * 4 independent 32x32x16 bf16 MFMAs and nothing else:
 * blocks * 8 * iters * 4 * 32768 flop.  Timed by the caller, it gives the rate the matrix pipes
 * sustain on this chip under a pure matrix load, hence the clock it holds there (rate / published
 * peak * nominal clock).  `out` receives blocks * 512 floats (so the work cannot be optimised away). */
int tritt_probe_mfma(float* out, int blocks, int iters, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRITTENTION_HIP_H */
