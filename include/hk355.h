/*
 * hk355 — C ABI of the MI355X (gfx950) quantized-contraction library.
 *
 * Every entry point:
 *   - takes plain device pointers owned by the caller (inputs and outputs are
 *     caller-allocated, as in the reference's pybind11 boundary, which only
 *     reads data_ptr()/shape: include/pyutils/pyutils.cuh:14-47, :66-71);
 *   - is asynchronous on `stream` (a hipStream_t passed as void*; NULL = the
 *     null stream, which is what the reference's bindings launch on:
 *     kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:24-32, :227-231);
 *   - returns HK_OK or a negative hk_status; it never aborts and never throws.
 *     Argument errors are detected on the host before anything is launched.
 */
#ifndef HK355_H
#define HK355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum hk_status {
    HK_OK = 0,
    HK_ERR_NULL_POINTER = -1, /* a required pointer is NULL                      */
    HK_ERR_BAD_SHAPE = -2,    /* a dimension is <= 0 or violates a divisibility  */
    HK_ERR_BAD_ALIGNMENT = -3,/* a pointer is not 16-byte aligned                */
    HK_ERR_WORKSPACE = -4,    /* workspace missing or too small                  */
    HK_ERR_LAUNCH = -5,       /* HIP reported an error at launch                 */
    HK_ERR_UNSUPPORTED = -6   /* valid but not implemented for these parameters  */
} hk_status;

/* Human-readable name of a status code (static storage). */
const char* hk_status_string(int status);

/* Library version, e.g. 100 = 0.1.0 (no reference counterpart). */
int hk_version(void);

/*
 * FP8 e4m3 (OCP e4m3fn) GEMM:  C[M,N] = bf16( (scale_a*scale_b) * sum_k A[m,k]*B[n,k] ).
 * A is [M,K] row-major, B is [N,K] row-major ("column-major B"), both 1 byte per
 * element; fp32 accumulation; C is [M,N] row-major bf16, rounded to nearest even.
 * Replaces the reference's FP8 GEMM executable (kernels/gemm/fp8fp32/README.md:7-21;
 * math = mma_ABt, include/ops/warp/register/tile/mma.cuh:382-422 with the fp8
 * MFMA of :112-125) behind the dispatch_micro(A, B, C) convention of
 * kernels/gemm/bf16fp32/mi350x/test_python.py:80-82. The reference applies no
 * scale; scale_a = scale_b = 1 reproduces it.
 * Requirements: M,N,K > 0; K % 16 == 0; A, B, C 16-byte aligned.
 */
int hk_fp8_gemm(const void* A_e4m3, const void* B_e4m3, void* C_bf16,
                int M, int N, int K, float scale_a, float scale_b, void* stream);

/* Same contract, forced onto one kernel variant (for tests and tuning):
 * 0 = portable kernel (any shape), 1 = 256x256x128 tile, 8 waves, 2 = 256x256x128 tile,
 * 4 waves, hand-interleaved schedule, 3 = 256x256x128 tile, 4 waves, plain loop.
 * Variants 1-3 need K % 128 == 0. */
int hk_fp8_gemm_variant(const void* A_e4m3, const void* B_e4m3, void* C_bf16,
                        int M, int N, int K, float scale_a, float scale_b,
                        int variant, void* stream);

/*
 * MXFP4 GEMM (OCP Microscaling v1.0): C[M,N] = bf16( sum_k a[m,k] * b[n,k] ) with
 *   a[m,k] = e2m1(A[m, k/2] nibble k%2; low nibble = even k) * 2^(A_scales[m, k/32] - 127)
 * and b likewise. A is [M, K/2] bytes, A_scales [M, K/32] e8m0 bytes, B [N, K/2], B_scales
 * [N, K/32], all row-major; fp32 accumulation, C [M,N] bf16 (RNE).
 * No counterpart in the reference (it has no MXFP4 code); same calling convention as
 * hk_fp8_gemm. Requirements: M,N,K > 0; K % 32 == 0; A, B, C 16-byte aligned.
 */
int hk_mxfp4_gemm(const void* A_e2m1, const void* A_scales_e8m0, const void* B_e2m1,
                  const void* B_scales_e8m0, void* C_bf16, int M, int N, int K, void* stream);

/* Same contract on a chosen kernel: 0 = portable kernel (any shape), 1 = 256x256x256 tile
 * kernel (needs K % 256 == 0 and 4-byte aligned scale pointers). */
int hk_mxfp4_gemm_variant(const void* A_e2m1, const void* A_scales_e8m0, const void* B_e2m1,
                          const void* B_scales_e8m0, void* C_bf16, int M, int N, int K,
                          int variant, void* stream);

/* ------------------------------------------------------------------ MoE routing
 * The reference has no MoE code; these entry points have no counterpart in it. They follow
 * the same conventions as the GEMMs (caller-owned device buffers, asynchronous, status code).
 * Integer outputs are deterministic: ties go to the lower expert id and the sort is stable.
 */

/* Top-k softmax routing. logits [T,E] fp32 -> ids [T,k] int32 (descending logit order) and
 * w [T,k] fp32 = softmax over the k selected logits. Requirements: k <= 64, E <= 512. */
int hk_moe_topk_softmax(const float* logits, int T, int E, int k, int32_t* ids, float* w,
                        void* stream);

/* Group-limited sigmoid routing (DeepSeek-V3 style). s = sigmoid(logit); selection score
 * c = s + bias (bias [E] may be NULL); experts form n_group contiguous groups; a group's score
 * is the sum of its two largest c; the topk_group best groups are kept; ids = top-k of c within
 * kept groups; w = s[ids] / sum(s[ids]) * routed_scale.
 * Requirements: E % n_group == 0, n_group <= 64, k <= topk_group * (E / n_group). */
int hk_moe_topk_grouped_sigmoid(const float* logits, const float* bias_or_null, int T, int E,
                                int k, int n_group, int topk_group, float routed_scale,
                                int32_t* ids, float* w, void* stream);

/* Stable sort of the T*k (token, choice) slots by expert id.
 * sorted_slots [T*k]: slot indices t*k+j ordered by expert, ascending slot index inside an
 * expert; expert_offsets [E+1]: exclusive prefix sum of per-expert counts; slot_to_pos [T*k]
 * (optional): position of each slot in sorted_slots. workspace: hk_moe_sort_workspace_bytes().
 * Requirements: E <= 512. */
size_t hk_moe_sort_workspace_bytes(int T, int k, int E);
int hk_moe_sort(const int32_t* ids, int T, int k, int E, int32_t* sorted_slots,
                int32_t* expert_offsets, int32_t* slot_to_pos_or_null, void* workspace,
                size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HK355_H */
