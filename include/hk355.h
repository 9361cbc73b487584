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

/* Tile (256, 128 or 64) that hk_fp8_gemm / hk_bf16_gemm / hk_mxfp4_gemm (format 0 / 1 / 2) pick for a shape
 * on the current device when the tile kernels can take it; consult_table 0: the rule alone, without the
 * generated per-shape table (what the sweep that writes the table compares against). Negative: a status.
 * Counterpart of the reference's per-shape solution selection
 * (analysis/baselines/gemm/utils/solution_selection.py, tuned.yaml). With at most 64 rows of A the FP8 and BF16
 * entry points may take the skinny kernel instead of a tile kernel (see hk_fp8_gemm_variant, 8); this function
 * reports the tile they would take otherwise. */
int hk_gemm_tile_choice(int format, int M, int N, int K, int consult_table);

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

/* The same GEMM with an optional workspace, for decode-like shapes (at most one 64x64 tile of C for
 * every second CU and K >= 6144, e.g. M = 128 with N = 4096, K = 8192): the K range is split over several workgroups per
 * tile, which write fp32 partial sums to the workspace, and a second kernel adds them in a fixed
 * order (deterministic) and rounds to bf16. hk_fp8_gemm_workspace_bytes returns the bytes this
 * needs, or 0 when the shape would not be split; with a NULL or too small workspace, or such a
 * shape, the call is hk_fp8_gemm. With at most 64 rows of A most such shapes go to the skinny kernel
 * (variant 8), which adds its partial sums inside the workgroup and leaves the workspace untouched.
 * No counterpart in the reference (compile-time shapes only). */
size_t hk_fp8_gemm_workspace_bytes(int M, int N, int K);
int hk_fp8_gemm_ws(const void* A_e4m3, const void* B_e4m3, void* C_bf16, int M, int N, int K,
                   float scale_a, float scale_b, void* workspace, size_t workspace_bytes, void* stream);

/* hk_fp8_gemm_ws without a workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart
 * in the reference. The split-K partial sums go to a file-scope device array of
 * hk_fp8_gemm_static_ws_max_bytes() = 8 MiB inside the library, which every GPU the library runs on
 * holds until the process ends; the call allocates and frees nothing. The first call on a device looks
 * the array's address up (make it before a capture starts). Shapes that the split-K path does not take
 * run as hk_fp8_gemm; a shape whose partial sums exceed the array returns HK_ERR_WORKSPACE (cannot
 * happen on a 256-CU device: at most 512 workgroups x 16 KiB). Results are bit-identical to
 * hk_fp8_gemm_ws. All calls on one GPU share the one array: calls that overlap in time on the same GPU
 * (different streams or threads) race and must be serialized by the caller. */
size_t hk_fp8_gemm_static_ws_max_bytes(void);
int hk_fp8_gemm_static_ws(const void* A_e4m3, const void* B_e4m3, void* C_bf16, int M, int N, int K,
                          float scale_a, float scale_b, void* stream);

/* Same contract, forced onto one kernel variant (for tests and tuning):
 * 0 = portable kernel (any shape), 1 = 256x256x128 tile, 8 waves in two ping-pong groups (the
 * reference's second FP8 schedule, kernels/gemm/fp8fp32/README.md:3-5, schedule of
 * kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:73-155), 4 = 256x256x128 tile, 4 waves,
 * hand-interleaved schedule over a five-slot LDS ring with the loads spread over the whole K-step
 * (what hk_fp8_gemm picks for large problems: the tile with the smallest estimated time, see
 * hk_gemm_tile_choice), 5 = 128x128x128 tile, 4
 * waves, plain loop over three LDS stages (picked for smaller problems), 6 = the same loop with
 * 64x64 tiles and four stages, two workgroups per CU (picked for the smallest), 7 = 192x256x128
 * tile, sixteen waves: four producers that only issue the
 * global->LDS loads and twelve consumers that only multiply (the wave-specialised structure of the
 * reference's kernels/gemm/bf16fp32/mi350x/micros/producer_consumer/32x16/micro_04_2stage_12c4p.cpp;
 * measured, not picked by default), 8 = the skinny kernel for M <= 64 (HK_ERR_UNSUPPORTED above): a
 * workgroup owns 32 rows of B and all rows of A, its waves split K among themselves, stream their pieces
 * of both operands through LDS stages of their own and add their partial sums in wave order
 * (deterministic; one pass over B at HBM speed, no workspace; picked for decode shapes: up to 32 rows
 * while N / 32 is at most the CU count, up to 16 rows at any N when K >= 4096, up to 64 rows while N / 32
 * is at most the CU count; 16 rows of B per workgroup while 32 would leave half of the CUs without one, B
 * loaded with the non-temporal hint from 8 MB of B on; no counterpart in the reference, whose shapes are
 * compile-time squares). 2 and 3 are not in use
 * (HK_ERR_UNSUPPORTED). All kernels zero-fill the last K-step of any K % 16 == 0; the tile kernels
 * (1, 4 - 7) give identical bits, the skinny kernel adds in another order. */
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
 * kernel (4 waves, hand-interleaved), 2 = 128x128 tiles / three LDS stages, 3 = 64x64 tiles / four
 * stages (the small-tile kernels of the FP8 GEMM with the scaled FP4 MFMA; hk_mxfp4_gemm picks by tile
 * count as hk_fp8_gemm does), 4 = 256x256x256 tile kernel with the 8-wave ping-pong schedule, 5 =
 * 192x256x256 tile producer / consumer kernel (see hk_fp8_gemm_variant, 7), 6 = the skinny kernel for M <= 64
 * (see hk_fp8_gemm_variant, 8; the scales travel like the operands, 128 bytes of a row at a time; picked by
 * hk_mxfp4_gemm, _pitched and _ws up to 64 rows while N / 32 is at most twice the CU count, up to 32 rows at any
 * N when K >= 8192). 1-3 take dense scale rows of
 * any K >= 512 (K % 32 == 0) and any alignment, 6 scale rows of any K, pitch and alignment; 4 and 5 need
 * K % 256 == 0 and 4-byte aligned scale pointers. */
int hk_mxfp4_gemm_variant(const void* A_e2m1, const void* A_scales_e8m0, const void* B_e2m1,
                          const void* B_scales_e8m0, void* C_bf16, int M, int N, int K,
                          int variant, void* stream);

/* The same GEMM with padded scale rows: row m of A_scales starts at A_scales + m * a_scale_pitch
 * bytes (pitch >= K / 32), likewise B_scales. With pitches that are multiples of 8 bytes and
 * 4-byte aligned scale pointers the tile kernel takes any K % 32 == 0 (the hidden size 2880 of
 * the MoE models: K / 32 = 90 scale bytes in rows of 96); in its last K-step the bytes past the
 * end of a row are not fetched and count as zeros, so the padding scale bytes only must not be
 * 0xFF (NaN). Other pitches go to the portable kernel. No counterpart in the reference. */
int hk_mxfp4_gemm_pitched(const void* A_e2m1, const void* A_scales_e8m0, int a_scale_pitch,
                          const void* B_e2m1, const void* B_scales_e8m0, int b_scale_pitch,
                          void* C_bf16, int M, int N, int K, void* stream);

/* The MXFP4 GEMM (scale rows with pitches, as hk_mxfp4_gemm_pitched; dense rows: pitch K / 32) with an
 * optional workspace for decode-like shapes, as hk_fp8_gemm_ws: few 64x64 tiles (at most a quarter of
 * what fills the GPU) and a K of at least 16 K-steps of 256 elements are split along K into fp32 partial
 * sums, added in a fixed order, when the shorter K loops save more time than the partial sums cost.
 * hk_mxfp4_gemm_workspace_bytes returns 0 for shapes that would not be split; without a (large enough,
 * 16-byte aligned) workspace, or with scale rows the tile kernels do not take, the call is
 * hk_mxfp4_gemm_pitched. No counterpart in the reference. */
size_t hk_mxfp4_gemm_workspace_bytes(int M, int N, int K);
int hk_mxfp4_gemm_ws(const void* A_e2m1, const void* A_scales_e8m0, int a_scale_pitch, const void* B_e2m1,
                     const void* B_scales_e8m0, int b_scale_pitch, void* C_bf16, int M, int N, int K,
                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * BF16 GEMM: C[M,N] = bf16( A[M,K] * B[N,K]^T ), A and B row-major bf16, fp32 accumulation, RNE.
 * Replaces the reference's flagship kernel behind tk_kernel.dispatch_micro(A, B, C)
 * (kernels/gemm/bf16fp32/mi350x/test_python.py:80-82, kernel kernels/gemm/bf16fp32/mi350x/, tile
 * and binding as in kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:13-42, 227-237), for any shape
 * instead of one compiled-in size. Requirements: M,N,K > 0; K % 8 == 0; A, B, C 16-byte aligned.
 */
int hk_bf16_gemm(const void* A_bf16, const void* B_bf16, void* C_bf16, int M, int N, int K,
                 void* stream);

/* The BF16 GEMM with an optional workspace for decode-like shapes, exactly as hk_fp8_gemm_ws:
 * few 64x64 tiles and a long K (at least 48 K-steps of 64 elements) are split along K into fp32
 * partial sums, added in a fixed order. hk_bf16_gemm_workspace_bytes returns 0 for shapes that
 * would not be split; without a (large enough) workspace the call is hk_bf16_gemm. */
size_t hk_bf16_gemm_workspace_bytes(int M, int N, int K);
int hk_bf16_gemm_ws(const void* A_bf16, const void* B_bf16, void* C_bf16, int M, int N, int K,
                    void* workspace, size_t workspace_bytes, void* stream);

/* Same contract on a chosen kernel: 0 = portable kernel (any shape), 1 = 256x256x64 tile kernel
 * (the FP8 ring schedule; the last K-step of a K that is not a multiple of 64 is zero-filled),
 * 2 = 128x128 tiles / three LDS stages, 3 = 64x64 tiles / four stages (the FP8 GEMM's small-tile
 * kernels with the bf16 MFMA; hk_bf16_gemm picks them by tile count as hk_fp8_gemm does), 4 = 256x256x64
 * tile kernel with the reference's 8-wave ping-pong schedule
 * (kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:73-155), 5 = 192x256x64 tile producer / consumer kernel
 * (kernels/gemm/bf16fp32/mi350x/micros/producer_consumer/32x16/micro_04_2stage_12c4p.cpp: four waves load,
 * twelve multiply), 6 = the skinny kernel for M <= 64 (see hk_fp8_gemm_variant, 8; picked by hk_bf16_gemm and
 * hk_bf16_gemm_ws under the same conditions). */
int hk_bf16_gemm_variant(const void* A_bf16, const void* B_bf16, void* C_bf16, int M, int N, int K,
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
 * Slots whose id lies outside [0, E) (e.g. -1 for a masked or padded token) take no part: they are
 * not counted, the valid slots fill sorted_slots[0 .. expert_offsets[E]) and the entries of
 * sorted_slots behind that, like slot_to_pos of the dropped slots, are left untouched.
 * Requirements: E <= 512. */
size_t hk_moe_sort_workspace_bytes(int T, int k, int E);
int hk_moe_sort(const int32_t* ids, int T, int k, int E, int32_t* sorted_slots,
                int32_t* expert_offsets, int32_t* slot_to_pos_or_null, void* workspace,
                size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ MXFP4 fused MoE
 * No counterpart in the reference. Tensors (all row-major, caller owned):
 *   x            [T, H]  bf16 activations
 *   w13          [E, 2I, H/2] packed e2m1; rows 0..I-1 = gate projection, I..2I-1 = up projection
 *   w13_scales   [E, 2I, w13_scale_pitch] e8m0, one per 32 elements of H; the pitch is >= H/32
 *                and a multiple of 8, padding bytes must not be 0xFF (use 127)
 *   w2           [E, H, I/2] packed e2m1, w2_scales [E, H, w2_scale_pitch] likewise over I
 *   y            [T, H]  bf16
 * Per token t and choice j with expert e = ids[t,j]:
 *   h = silu(xq W13g[e]^T) * (xq W13u[e]^T),  o = hq W2[e]^T,  y[t] = sum_j w[t,j] * bf16(o)
 * where xq / hq are the activations re-quantized to MXFP4 (blocks of 32 along H / I, OCP MX
 * rule: shared exponent floor(log2(amax)) - 2), so every GEMM runs on the FP4 MFMA path.
 * Requirements: H % 32 == 0, I % 32 == 0, E <= 512, k <= 64.
 */

/* bf16 [rows, cols] -> packed e2m1 [rows, cols/2] + e8m0 scales [rows, scale_pitch]
 * (scale_pitch >= cols/32, multiple of 8; padding columns are written as 127). */
int hk_mxfp4_quantize_rows(const void* x_bf16, int rows, int cols, void* packed, void* scales,
                           int scale_pitch, void* stream);

/* y[t,:] = bf16(sum_j w[t,j] * o[slot_to_pos[t*k+j], :]), o [T*k, H] bf16. H % 8 == 0.
 * A position outside [0, T*k) is not read and adds nothing to its token. */
int hk_moe_unpermute(const void* o_bf16, const float* w, const int32_t* slot_to_pos, int T, int k,
                     int H, void* y_bf16, void* stream);
/* As hk_moe_unpermute with a residual: y[t,:] = bf16(add[t,:] + sum_j ...), add [T, H] bf16 or NULL
 * (e.g. the output of a shared expert that every token passes through). */
int hk_moe_unpermute_add(const void* o_bf16, const float* w, const int32_t* slot_to_pos, int T, int k,
                         int H, const void* add_bf16_or_null, void* y_bf16, void* stream);

/* Bytes of workspace a layer of this shape needs; 0 for a shape the entry points refuse with
 * HK_ERR_BAD_SHAPE (the other hk_moe_*_workspace_bytes functions likewise). */
size_t hk_moe_mxfp4_workspace_bytes(int T, int H, int I, int E, int k);

/* Offline weight pre-shuffle (weight_layout = 1 below). For every expert, n-tile and K-step the
 * 256 x 128-byte weight tile is stored contiguously in the order the kernel keeps it in LDS
 * (K zero-padded to whole 256-element steps), scales likewise as 256 x 8-byte tiles, so that the
 * GEMMs stream weights from HBM in 32 KiB bursts. mode 0: gate+up matrix [E, 2N, K/2] with N = I,
 * K = H; mode 1: down matrix [E, N, K/2] with N = H, K = I; mode 2: as mode 0 for a source with
 * interleaved gate / up rows (2c / 2c + 1), same output format. scales [E, rows, scale_pitch]. */
int hk_moe_mxfp4_preshuffle_bytes(int E, int N, int K, int mode, size_t* w_bytes, size_t* s_bytes);
int hk_moe_mxfp4_preshuffle(const void* w, const void* scales, int scale_pitch, int E, int N, int K,
                            int mode, void* out_w, void* out_s, void* stream);

/* Expert MLP for tokens that are already routed and sorted (outputs of hk_moe_topk_* and
 * hk_moe_sort): activation quantization, grouped gate+up GEMM with SiLU-mul and MX
 * re-quantization, grouped down GEMM, weighted un-permute. weight_layout 0: w13 / w2 and their
 * scales in the plain row-major layout above; 1: outputs of hk_moe_mxfp4_preshuffle (the scale
 * pitch arguments are then ignored). Both layouts give bit-identical results. sorted_slots,
 * expert_offsets and slot_to_pos must be one consistent result of hk_moe_sort: the kernels index
 * activations and outputs with them (through range-checked descriptors where they fetch rows by
 * token, so slots outside [0, T*k) read zeros or neighbouring workspace, never outside it; the
 * un-permute skips positions outside [0, T*k)). */
int hk_moe_mxfp4_experts(const void* x_bf16, const void* w13, const void* w13_scales,
                         int w13_scale_pitch, const void* w2, const void* w2_scales,
                         int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                         const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                         int T, int H, int I, int E, int k, int weight_layout, void* workspace,
                         size_t workspace_bytes, void* stream);

/* Whole layer: top-k softmax routing of router_logits [T,E] fp32, sort, expert MLP. */
int hk_moe_mxfp4_forward(const void* x_bf16, const float* router_logits, const void* w13,
                         const void* w13_scales, int w13_scale_pitch, const void* w2,
                         const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H, int I,
                         int E, int k, int weight_layout, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Model-faithful variants of the two entry points above (no counterpart in the reference; the
 * formulas follow the published GPT-OSS model code):
 *   bias13 [E, 2I] fp32 or NULL: added to the gate+up GEMM result before the activation
 *   bias2  [E, H]  fp32 or NULL: added to the down GEMM result before the weighted sum
 *   activation 0: silu(gate) * up; 1: clamped SwiGLU, g = min(gate, limit), u = clamp(up, +-limit),
 *              h = (u + 1) * g * sigmoid(alpha * g)   (GPT-OSS: alpha 1.702, limit 7)
 *   w13_interleaved != 0: gate / up of h column c are rows 2c / 2c + 1 of w13, w13_scales and
 *              bias13 instead of rows c / I + c. With weight_layout 1 the weights must have been
 *              shuffled with mode 2 (hk_moe_mxfp4_preshuffle), which reads that row order.
 * With all options off they run the same kernels as the plain entry points. */
int hk_moe_mxfp4_experts_ex(const void* x_bf16, const void* w13, const void* w13_scales,
                            int w13_scale_pitch, const void* w2, const void* w2_scales,
                            int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                            const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                            int T, int H, int I, int E, int k, int weight_layout, const float* bias13,
                            const float* bias2, int activation, float alpha, float limit,
                            int w13_interleaved, void* workspace, size_t workspace_bytes, void* stream);
int hk_moe_mxfp4_forward_ex(const void* x_bf16, const float* router_logits, const void* w13,
                            const void* w13_scales, int w13_scale_pitch, const void* w2,
                            const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H, int I,
                            int E, int k, int weight_layout, const float* bias13, const float* bias2,
                            int activation, float alpha, float limit, int w13_interleaved,
                            void* workspace, size_t workspace_bytes, void* stream);

/* The same layer with MXFP8 activations (W4A8; no counterpart in the reference): x and h are
 * re-quantized to e4m3 elements with one e8m0 scale per 32 (OCP MX rule: shared exponent
 * floor(log2(amax)) - 8, elements rounded to nearest even and saturated at +-448) instead of e2m1,
 * and the grouped GEMMs run the mixed MFMA (fp4 weights x fp8 activations). Weights must be in
 * the pre-shuffled layout (outputs of hk_moe_mxfp4_preshuffle); the other arguments are those of
 * hk_moe_mxfp4_experts_ex / hk_moe_mxfp4_forward_ex. The workspace is larger than for MXFP4
 * activations (256 bytes per row and K-step): hk_moe_mxfp4_a8_workspace_bytes. */
int hk_mxfp8_quantize_rows(const void* x_bf16, int rows, int cols, void* codes_e4m3, void* scales,
                           int scale_pitch, void* stream);
size_t hk_moe_mxfp4_a8_workspace_bytes(int T, int H, int I, int E, int k);
int hk_moe_mxfp4_a8_experts(const void* x_bf16, const void* w13_shuffled, const void* w13_scales_shuffled,
                            const void* w2_shuffled, const void* w2_scales_shuffled, const float* topk_w,
                            const int32_t* sorted_slots, const int32_t* expert_offsets,
                            const int32_t* slot_to_pos, void* y_bf16, int T, int H, int I, int E, int k,
                            const float* bias13, const float* bias2, int activation, float alpha, float limit,
                            int w13_interleaved, void* workspace, size_t workspace_bytes, void* stream);
int hk_moe_mxfp4_a8_forward(const void* x_bf16, const float* router_logits, const void* w13_shuffled,
                            const void* w13_scales_shuffled, const void* w2_shuffled,
                            const void* w2_scales_shuffled, void* y_bf16, int T, int H, int I, int E, int k,
                            const float* bias13, const float* bias2, int activation, float alpha, float limit,
                            int w13_interleaved, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------- FP8 block-scaled fused MoE
 * No counterpart in the reference. DeepSeek-V3 style quantization:
 *   x          [T, H] e4m3, x_scales [T, H/128] fp32 (one scale per 1 x 128 block: x ~ q * s)
 *   w13        [E, 2I, H] e4m3 (rows 0..I-1 gate, I..2I-1 up), w13_scales [E, 2I/128, H/128] fp32
 *   w2         [E, H, I] e4m3, w2_scales [E, H/128, I/128] fp32 (one scale per 128 x 128 block)
 *   y          [T, H] bf16
 * h = silu(x W13g^T) * (x W13u^T) is re-quantized to e4m3 with 1 x 128 scales (scale = amax/448),
 * o = h W2^T, y[t] = sum_j w[t,j] * bf16(o). Requirements: H % 128 == 0, I % 128 == 0,
 * E <= 512, k <= 64.
 */

/* bf16 [rows, cols] -> e4m3 [rows, cols] + fp32 scales [rows, cols/128], scale = amax/448
 * (1 for an all-zero block), elements round to nearest even, saturating. cols % 128 == 0. */
int hk_fp8_quantize_rows_1x128(const void* x_bf16, int rows, int cols, void* q_e4m3, float* scales,
                               void* stream);

size_t hk_moe_fp8blk_workspace_bytes(int T, int H, int I, int E, int k);

/* Expert MLP for routed and sorted tokens (outputs of hk_moe_topk_* and hk_moe_sort). */
int hk_moe_fp8blk_experts(const void* x_e4m3, const float* x_scales, const void* w13,
                          const float* w13_scales, const void* w2, const float* w2_scales,
                          const float* topk_w, const int32_t* sorted_slots,
                          const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                          int T, int H, int I, int E, int k, void* workspace, size_t workspace_bytes,
                          void* stream);

/* Whole layer with group-limited sigmoid routing (see hk_moe_topk_grouped_sigmoid). */
int hk_moe_fp8blk_forward(const void* x_e4m3, const float* x_scales, const float* router_logits,
                          const float* router_bias_or_null, int n_group, int topk_group,
                          float routed_scale, const void* w13, const float* w13_scales, const void* w2,
                          const float* w2_scales, void* y_bf16, int T, int H, int I, int E, int k,
                          void* workspace, size_t workspace_bytes, void* stream);

/* The two entry points above with a residual y_add [T, H] bf16 (or NULL) that is added, in fp32,
 * to the weighted sum of the routed experts before the single bf16 rounding: the DeepSeek-V3
 * shared expert. Its output is computed with hk_moe_fp8blk_experts on trivial routing (E = 1,
 * k = 1, weight 1, identity order), then passed here. y_add may alias y_bf16. */
int hk_moe_fp8blk_experts_ex(const void* x_e4m3, const float* x_scales, const void* w13,
                             const float* w13_scales, const void* w2, const float* w2_scales,
                             const float* topk_w, const int32_t* sorted_slots,
                             const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                             int T, int H, int I, int E, int k, const void* y_add_bf16_or_null,
                             void* workspace, size_t workspace_bytes, void* stream);
int hk_moe_fp8blk_forward_ex(const void* x_e4m3, const float* x_scales, const float* router_logits,
                             const float* router_bias_or_null, int n_group, int topk_group,
                             float routed_scale, const void* w13, const float* w13_scales,
                             const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                             int E, int k, const void* y_add_bf16_or_null, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Offline pre-shuffle of FP8 block-scaled expert weights (weight_layout = 1 below; no counterpart in
 * the reference). For every expert, tile of 256 weight rows and K-step of 128 columns the 32 KiB
 * weight tile is stored contiguously as the MFMA operand fragments of the kernel's four column waves
 * (1 KiB pieces in lane order), so that the grouped GEMMs load weights from HBM straight into MFMA
 * operand registers instead of staging them in LDS. mode 0: gate+up matrix [E, 2N, K] with N = I,
 * K = H; mode 1: down matrix [E, N, K] with N = H, K = I. The fp32 block scales keep their layout.
 * Requirements: N % 128 == 0, K % 128 == 0, w and out_w 16-byte aligned. */
int hk_moe_fp8blk_preshuffle_bytes(int E, int N, int K, int mode, size_t* w_bytes);
int hk_moe_fp8blk_preshuffle(const void* w, int E, int N, int K, int mode, void* out_w, void* stream);

/* hk_moe_fp8blk_experts_ex / hk_moe_fp8blk_forward_ex with a choice of weight layout: 0 = w13 / w2 in
 * the plain row-major layout, 1 = outputs of hk_moe_fp8blk_preshuffle (the scale tensors are the
 * plain ones in both cases). Both layouts give bit-identical results; layout 1 is the fast path. */
int hk_moe_fp8blk_experts_ex2(const void* x_e4m3, const float* x_scales, const void* w13,
                              const float* w13_scales, const void* w2, const float* w2_scales,
                              const float* topk_w, const int32_t* sorted_slots,
                              const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                              int T, int H, int I, int E, int k, int weight_layout,
                              const void* y_add_bf16_or_null, void* workspace, size_t workspace_bytes,
                              void* stream);
int hk_moe_fp8blk_forward_ex2(const void* x_e4m3, const float* x_scales, const float* router_logits,
                              const float* router_bias_or_null, int n_group, int topk_group,
                              float routed_scale, const void* w13, const float* w13_scales,
                              const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                              int E, int k, int weight_layout, const void* y_add_bf16_or_null,
                              void* workspace, size_t workspace_bytes, void* stream);

/* The whole layer from bf16 activations x [T, H]: every token is quantized once to e4m3 with 1 x 128
 * fp32 scales (hk_fp8_quantize_rows_1x128, into the workspace) ahead of the gather that repeats it
 * for its k experts, then hk_moe_fp8blk_forward_ex2. Same result as quantizing with
 * hk_fp8_quantize_rows_1x128 and calling hk_moe_fp8blk_forward_ex2. */
int hk_moe_fp8blk_forward_bf16(const void* x_bf16, const float* router_logits,
                               const float* router_bias_or_null, int n_group, int topk_group,
                               float routed_scale, const void* w13, const float* w13_scales,
                               const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                               int E, int k, int weight_layout, const void* y_add_bf16_or_null,
                               void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HK355_H */
