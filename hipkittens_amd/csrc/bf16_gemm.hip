// BF16 GEMM for gfx950: C[M,N] = bf16( A[M,K] * B[N,K]^T ), bf16 operands, fp32 accumulate.
//
// Counterpart of the reference's flagship kernel (kernels/gemm/bf16fp32/mi350x, bound as
// tk_kernel.dispatch_micro(A, B, C), kernels/gemm/bf16fp32/mi350x/test_python.py:80-82; tile
// 256x256x64, kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:13-42), built on this library's FP8
// skeleton to show that the schedule is independent of the operand type: a K-step is again
// 128 bytes per operand row (64 bf16 elements), so tile layout, swizzle, direct global->LDS
// loads, the five-slot LDS ring and the slot plan are those of the FP8 kernel (one body: gemm_ring.h); the
// two 16-byte halves a lane reads per fragment row are K elements 8g.. and 32 + 8g.. and feed
// two v_mfma_f32_16x16x32_bf16 (16 cycles each, together as long as one FP8 MFMA).
#include "gemm_tile.h"
#include "gemm_ring.h"
#include "gemm_small_tile.h"
#include "gemm_pingpong.h"
#include "gemm_prodcons.h"
#include "gemm_skinny.h"
#include "../../include/hk355.h"

namespace hk {

// acc(16x16) += X(16x32 bf16) * Y(16x32 bf16)^T with the accumulator tied in place in an AGPR;
// lane l supplies row l % 16, K elements 8 (l / 16) .. +8 of each operand.
__device__ __forceinline__ void mfma_bf16_16x16x32_acc(v4f& acc, const v4i& x, const v4i& y) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
}

// The 4-wave ring schedule (gemm_ring.h) with two bf16 MFMAs per fragment pair.
struct Bf16RingMma {
    struct Frag { v4i lo, hi; };  // K elements 8 g .. +8 and 32 + 8 g .. +8 of the lane's row
    static constexpr int kPasses = 2;
    static __device__ __forceinline__ Frag load(uint32_t lo, uint32_t hi, int imm) {
        Frag f;
        f.lo = *(lds_v4i_t*)(uintptr_t)(lo + imm);
        f.hi = *(lds_v4i_t*)(uintptr_t)(hi + imm);
        return f;
    }
    template <int PASS>
    static __device__ __forceinline__ void mma(v4f& acc, const Frag& b, const Frag& a) {
        if constexpr (PASS == 0) mfma_bf16_16x16x32_acc(acc, b.lo, a.lo);
        else mfma_bf16_16x16x32_acc(acc, b.hi, a.hi);
    }
    static __device__ __forceinline__ int raster_group(int band_n, int tiles_n) { return band_n < tiles_n ? 4 : 8; }
};
// STREAM_C: C is stored with the non-temporal hint; the host asks for it for large outputs of whole tiles while the
// operands fit the memory-side cache (launch_bf16_ring has the rule and the measurements; 8192^3: 1577 -> 1593
// TFLOP/s on one box, 1541 -> 1558 on another). (FP8 and MXFP4 at 8192^3: -1.0 / -1.5 %.)
template <bool EDGE, bool STREAM_C = false>
__global__ __launch_bounds__(256) void bf16_gemm_4wave_ring_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_ring_body<Bf16RingMma, EDGE, STREAM_C>(smem, A, B, C, M, N, 2 * K, alpha, tiles_m, tiles_n, band_n);
}


// Portable kernel for any M, N and K % 8 == 0: 4 waves, each a 32x32 patch of a 64x64 tile,
// operands fetched straight from global memory into MFMA fragments with per-lane masking.
__global__ __launch_bounds__(256) void bf16_gemm_portable_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha) {
    typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
    const int lane = lane_id(), w = wave_id();
    const int r = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.y * 64 + (w >> 1) * 32;
    const int col0 = blockIdx.x * 64 + (w & 1) * 32;
    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    auto frag = [&](const uint16_t* base, int row, int rows, int k0) {
        v4i v = {0, 0, 0, 0};
        if (row < rows && k0 + 8 * g < K) v = *(const v4i*)(base + (size_t)row * K + k0 + 8 * g);
        return __builtin_bit_cast(v8bf, v);
    };
    for (int k0 = 0; k0 < K; k0 += 32) {
        v8bf af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            af[i] = frag(A, row0 + 16 * i + r, M, k0);
            bf[i] = frag(B, col0 + 16 * i + r, N, k0);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = row0 + 16 * i + r;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const v4f x = acc[i][j] * alpha;
            const float v[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = col0 + 16 * j + 4 * g + e;
                if (row < M && col < N) C[(size_t)row * N + col] = (uint16_t)(pack_bf16(v[e], 0.f) & 0xffffu);
            }
        }
    }
}

// Small-tile kernels (gemm_small_tile.h) with the bf16 MFMA: the two 16-byte halves of a fragment
// row are K elements 8g.. and 32 + 8g.. of the 64-element K-step, one v_mfma_f32_16x16x32_bf16 each.
struct Bf16Mma {
    static constexpr bool kScaled = false;
    typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ void mma(v4f& acc, const v8i& b, const v8i& a) {
        const v4i blo = {b[0], b[1], b[2], b[3]}, bhi = {b[4], b[5], b[6], b[7]};
        const v4i alo = {a[0], a[1], a[2], a[3]}, ahi = {a[4], a[5], a[6], a[7]};
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, blo), __builtin_bit_cast(v8bf, alo),
                                                      acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, bhi), __builtin_bit_cast(v8bf, ahi),
                                                      acc, 0, 0, 0);
    }
};
// K: the operands' row length in bytes (2 bytes per element).
template <int TILE, int STAGES, bool EDGE, bool SPLIT>
__global__ __launch_bounds__(256) void bf16_gemm_small_tile_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int kps, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_small_tile_body<Bf16Mma, TILE, STAGES, EDGE, SPLIT>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n, kps,
                                                             partial);
}

// 8-wave ping-pong kernel (gemm_pingpong.h) with the bf16 MFMA: the schedule of the reference's flagship
// kernel (kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:73-155). K: the operands' row length in bytes.
template <bool EDGE>
__global__ __launch_bounds__(512) void bf16_gemm_pingpong_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_pingpong_body<Bf16Mma, EDGE>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n, band_n);
}

template <bool EDGE>
static int launch_bf16_pingpong(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream) {
    auto kern = bf16_gemm_pingpong_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPpLdsBytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(512), kPpLdsBytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, 2 * K, 1.0f, tiles_m, tiles_n,
                       raster_band(((long long)M + N) * K * 2, tiles_n));
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// Producer / consumer kernel (gemm_prodcons.h) with the bf16 MFMA: the reference's wave-specialised micro kernel
// (kernels/gemm/bf16fp32/mi350x/micros/producer_consumer/32x16/micro_04_2stage_12c4p.cpp) on this library's tile
// format. K: the operands' row length in bytes.
template <bool EDGE>
__global__ __launch_bounds__(kPcThreads) void bf16_gemm_prodcons_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_prodcons_body<Bf16Mma, EDGE>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n);
}

template <bool EDGE>
static int launch_bf16_prodcons(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream) {
    auto kern = bf16_gemm_prodcons_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPcLdsBytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + kPcBM - 1) / kPcBM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kPcThreads), kPcLdsBytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, 2 * K, 1.0f, tiles_m, tiles_n);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// The skinny kernel (gemm_skinny.h) with the BF16 MFMA. K: the operands' row length in bytes.
template <int R, int NW, int D, int NF, bool NT>
__global__ __launch_bounds__(64 * NW) void bf16_gemm_skinny_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_skinny_body<Bf16Mma, R, NW, D, NF, NT>(smem, A, B, C, M, N, K, alpha);
}
static int launch_bf16_skinny(const void* A, const void* B, void* C, int M, int N, int K_elems, hipStream_t stream) {
    const int K = 2 * K_elems;
    const float alpha = 1.0f;
    HK_SKINNY_DISPATCH(bf16_gemm_skinny_kernel);
}

template <int TILE, int STAGES, bool EDGE>
static int launch_bf16_small_tile(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream) {
    auto kern = bf16_gemm_small_tile_kernel<TILE, STAGES, EDGE, false>;
    constexpr int lds_bytes = STAGES * 2 * TILE * BK;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + TILE - 1) / TILE, tiles_n = (N + TILE - 1) / TILE;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, 2 * K, 1.0f, tiles_m, tiles_n, 0, (float*)nullptr);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <bool EDGE>
static int launch_bf16_splitk(const void* A, const void* B, void* C, int M, int N, int K, int splits, float* partial,
                              hipStream_t stream) {
    static DeviceOnce configured;
    return launch_small_tile_splitk(bf16_gemm_small_tile_kernel<kTinyTile, kTinyStages, EDGE, true>, configured, A,
                                    B, C, M, N, 2 * K, 1.0f, splits, partial, stream);
}

template <bool EDGE, bool STREAM_C>
static int launch_bf16_ring_kernel(const void* A, const void* B, void* C, int M, int N, int K, int band_n,
                                  hipStream_t stream) {
    auto kern = bf16_gemm_4wave_ring_kernel<EDGE, STREAM_C>;
    constexpr int lds_bytes = 5 * kTileBytes;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, K, 1.0f, tiles_m, tiles_n, band_n);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}
template <bool EDGE>
static int launch_bf16_ring(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream) {
    const int tiles_n = (N + BN - 1) / BN;
    const int band_n = raster_band(((long long)M + N) * K * 2, tiles_n);
    // whole tiles, operands that fit the memory-side cache (no bands) and a C of 96 MB or more: C goes out with the
    // non-temporal hint (8192^3: +0.7 to 1.2 %; 4096^3, a C of 32 MB: -1.2 %; 16384^3, banded: -0.75 %)
    if constexpr (!EDGE)
        if (band_n >= tiles_n && (long long)M * N * 2 >= (96ll << 20))
            return launch_bf16_ring_kernel<false, true>(A, B, C, M, N, K, band_n, stream);
    return launch_bf16_ring_kernel<EDGE, false>(A, B, C, M, N, K, band_n, stream);
}

}  // namespace hk

extern "C" int hk_bf16_gemm_variant(const void* A, const void* B, void* C, int M, int N, int K, int variant,
                                    void* stream) {
    using namespace hk;
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 8) != 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (variant < 0 || variant > 6) return HK_ERR_UNSUPPORTED;
    if (variant == 6 && M > kSkinnyMaxM) return HK_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (variant == 0) {
        if ((long long)((M + 63) / 64) > 65535) return HK_ERR_BAD_SHAPE;
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        hipLaunchKernelGGL(bf16_gemm_portable_kernel, grid, dim3(256), 0, s, (const uint16_t*)A,
                           (const uint16_t*)B, (uint16_t*)C, M, N, K, 1.0f);
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    if ((long long)2 * K * BM >= (1ll << 31)) return HK_ERR_BAD_SHAPE;
    if (variant == 6) return launch_bf16_skinny(A, B, C, M, N, K, s);
    if (variant == 2) {
        const bool edge128 = (M % kSmallTile) != 0 || (N % kSmallTile) != 0;
        return edge128 ? launch_bf16_small_tile<kSmallTile, kSmallStages, true>(A, B, C, M, N, K, s)
                       : launch_bf16_small_tile<kSmallTile, kSmallStages, false>(A, B, C, M, N, K, s);
    }
    if (variant == 3) {
        const bool edge64 = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
        return edge64 ? launch_bf16_small_tile<kTinyTile, kTinyStages, true>(A, B, C, M, N, K, s)
                      : launch_bf16_small_tile<kTinyTile, kTinyStages, false>(A, B, C, M, N, K, s);
    }
    if (variant == 5) {
        const bool e = (M % kPcBM) != 0 || (N % BN) != 0;
        return e ? launch_bf16_prodcons<true>(A, B, C, M, N, K, s) : launch_bf16_prodcons<false>(A, B, C, M, N, K, s);
    }
    const bool edge = (M % BM) != 0 || (N % BN) != 0;
    if (variant == 4)
        return edge ? launch_bf16_pingpong<true>(A, B, C, M, N, K, s) : launch_bf16_pingpong<false>(A, B, C, M, N, K, s);
    return edge ? launch_bf16_ring<true>(A, B, C, M, N, K, s) : launch_bf16_ring<false>(A, B, C, M, N, K, s);
}

extern "C" int hk_bf16_gemm(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
    using namespace hk;
    if (gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const bool tile_ok = K > 0 && (long long)2 * K * BM < (1ll << 31);
    // the same choice of tile as hk_fp8_gemm (pick_tile), with this format's measured corrections
    const int tile = pick_tile(kFmtBf16, M, N, (int)((2ll * K + BK - 1) / BK), kTileRuleBf16);
    const bool skinny = tile_ok && use_skinny(M, N, (int)((2ll * K + BK - 1) / BK), false, moe_num_compute_units());
    const int variant = !tile_ok ? 0 : skinny ? 6 : tile == kTinyTile ? 3 : tile == kSmallTile ? 2 : 1;
    return hk_bf16_gemm_variant(A, B, C, M, N, K, variant, stream);
}

extern "C" size_t hk_bf16_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || K >= (1 << 29) || hk::gemm_dims_too_large(M, N, K)) return 0;
    const int s = hk::splitk_ranges(M, N, 2 * K);
    return s < 2 ? 0 : (size_t)s * M * N * sizeof(float);
}

extern "C" int hk_bf16_gemm_ws(const void* A, const void* B, void* C, int M, int N, int K, void* workspace,
                               size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const int splits = K < (1 << 29) ? splitk_ranges(M, N, 2 * K) : 1;
    const bool can_split = splits >= 2 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) &&
                           (K % 8) == 0 && (long long)2 * K * BM < (1ll << 31) && (long long)M * N < (1ll << 40);
    if (!can_split) return hk_bf16_gemm(A, B, C, M, N, K, stream);
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)workspace) & 15u) return HK_ERR_BAD_ALIGNMENT;
    // the skinny kernel adds its partial sums inside the workgroup and leaves the workspace alone
    if (use_skinny(M, N, (int)((2ll * K + BK - 1) / BK), true, moe_num_compute_units()))
        return hk_bf16_gemm_variant(A, B, C, M, N, K, 6, stream);
    const bool edge = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
    return edge ? launch_bf16_splitk<true>(A, B, C, M, N, K, splits, (float*)workspace, (hipStream_t)stream)
                : launch_bf16_splitk<false>(A, B, C, M, N, K, splits, (float*)workspace, (hipStream_t)stream);
}
