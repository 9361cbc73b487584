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

#ifdef __cplusplus
}
#endif
#endif /* HK355_H */
