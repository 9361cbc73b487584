// FP8 e4m3 GEMM for gfx950: C[M,N] = bf16(alpha * A[M,K] * B[N,K]^T), fp32 accumulate.
//
// Replaces the reference's kernels/gemm/fp8fp32 executables (4-wave / 8-wave
// schedules, kernels/gemm/fp8fp32/README.md:3-21); helper layer studied:
// kernels/gemm/fp8fp32/FP8_4wave/utils.cpp:23-174.
//
// Tile kernels: one workgroup owns a 256x256 tile of C and walks K in steps of 128. A and B tiles
// (256 rows x 128 bytes each) are fetched with direct global->LDS loads into swizzled LDS tiles; each
// wave reads its operand fragments with ds_read_b128 and issues v_mfma_f32_16x16x128_f8f6f4. The MFMA
// is issued with the operand roles swapped (B rows as the "A" operand) so that a lane's 4 accumulator
// values are 4 consecutive columns of one C row, and the B tile's rows are permuted on their way into
// LDS so that two neighbouring MFMA tiles give a lane 8 consecutive columns = one 16-byte bf16 store.
// Two schedules, as in the reference: 4 waves with hand-interleaved slots (fp8_gemm_4wave_ring_kernel,
// the default) and 8 waves in two ping-pong groups (gemm_pingpong.h).
#include "gemm_tile.h"
#include "gemm_ring.h"
#include "gemm_small_tile.h"
#include "gemm_pingpong.h"
#include "gemm_prodcons.h"
#include "gemm_skinny.h"
#include "../../include/hk355.h"

namespace hk {

// ---------------------------------------------------------------------------------------
// The default kernel: the 4-wave ring schedule (gemm_ring.h) with the FP8 MFMA.
struct Fp8RingMma {
    using Frag = v8i;
    static constexpr int kPasses = 1;
    static __device__ __forceinline__ Frag load(uint32_t lo, uint32_t hi, int imm) { return lds_frag(lo, hi, imm); }
    template <int PASS>
    static __device__ __forceinline__ void mma(v4f& acc, const Frag& b, const Frag& a) {
        mfma_fp8_16x16x128_acc(acc, b, a);
    }
    static __device__ __forceinline__ int raster_group(int, int) { return 4; }
};
template <bool EDGE>
__global__ __launch_bounds__(256) void fp8_gemm_4wave_ring_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_ring_body<Fp8RingMma, EDGE>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n, band_n);
}

// ---------------------------------------------------------------------------------------
// Small-tile kernels (gemm_small_tile.h) with the FP8 MFMA.
struct Fp8Mma {
    static constexpr bool kScaled = false;
    static __device__ __forceinline__ void mma(v4f& acc, const v8i& b, const v8i& a) {
        acc = mfma_fp8_16x16x128(b, a, acc);
    }
};
// 8-wave ping-pong kernel (gemm_pingpong.h) with the FP8 MFMA: the reference's second FP8 schedule
// (kernels/gemm/fp8fp32/README.md:3-5).
template <bool EDGE>
__global__ __launch_bounds__(512) void fp8_gemm_pingpong_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_pingpong_body<Fp8Mma, EDGE>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n, band_n);
}

// Producer / consumer kernel (gemm_prodcons.h) with the FP8 MFMA: four waves that only load, twelve that only
// multiply (after the reference's micros/producer_consumer/32x16/micro_04_2stage_12c4p.cpp).
template <bool EDGE>
__global__ __launch_bounds__(kPcThreads) void fp8_gemm_prodcons_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_prodcons_body<Fp8Mma, EDGE>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n);
}

template <int TILE, int STAGES, bool EDGE, bool SPLIT>
__global__ __launch_bounds__(256) void fp8_gemm_small_tile_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int kps, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_small_tile_body<Fp8Mma, TILE, STAGES, EDGE, SPLIT>(smem, A, B, C, M, N, K, alpha, tiles_m, tiles_n, kps,
                                                            partial);
}

// Portable kernel for any M, N and K % 16 == 0: 4 waves, each a 32x32 patch of a 64x64
// tile, operands fetched straight from global memory into MFMA fragments with
// per-lane masking (rows past the edge and 16-byte chunks past K read as zero).
__global__ __launch_bounds__(256) void fp8_gemm_portable_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha) {
    const int lane = lane_id(), w = wave_id();
    const int r = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.y * 64 + (w >> 1) * 32;
    const int col0 = blockIdx.x * 64 + (w & 1) * 32;
    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto frag = [&](const uint8_t* base, int row, int rows, int k0) {
        v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
        if (row < rows) {
            const uint8_t* p = base + (size_t)row * K + k0 + 32 * g;
            if (k0 + 32 * g < K) lo = *(const v4i*)p;
            if (k0 + 32 * g + 16 < K) hi = *(const v4i*)(p + 16);
        }
        return (v8i)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };

    for (int k0 = 0; k0 < K; k0 += 128) {
        v8i af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            af[i] = frag(A, row0 + 16 * i + r, M, k0);
            bf[i] = frag(B, col0 + 16 * i + r, N, k0);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma_fp8_16x16x128(bf[j], af[i], acc[i][j]);
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
                if (row < M && col < N)
                    C[(size_t)row * N + col] = (uint16_t)(pack_bf16(v[e], 0.f) & 0xffffu);
            }
        }
    }
}

// The skinny kernel (gemm_skinny.h) with the FP8 MFMA.
template <int R, int NW, int D, int NF, bool NT>
__global__ __launch_bounds__(64 * NW) void fp8_gemm_skinny_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_skinny_body<Fp8Mma, R, NW, D, NF, NT>(smem, A, B, C, M, N, K, alpha);
}
static int launch_skinny(const void* A, const void* B, void* C, int M, int N, int K, float alpha, hipStream_t stream) {
    HK_SKINNY_DISPATCH(fp8_gemm_skinny_kernel);
}

template <bool EDGE>
static int launch_prodcons(const void* A, const void* B, void* C, int M, int N, int K, float alpha, hipStream_t stream) {
    auto kern = fp8_gemm_prodcons_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPcLdsBytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + kPcBM - 1) / kPcBM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kPcThreads), kPcLdsBytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha, tiles_m, tiles_n);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <bool EDGE>
static int launch_pingpong(const void* A, const void* B, void* C, int M, int N, int K, float alpha, hipStream_t stream) {
    auto kern = fp8_gemm_pingpong_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPpLdsBytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(512), kPpLdsBytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha, tiles_m, tiles_n,
                       raster_band(((long long)M + N) * K, tiles_n));
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <int TILE, int STAGES, bool EDGE>
static int launch_small_tile(const void* A, const void* B, void* C, int M, int N, int K, float alpha,
                             hipStream_t stream) {
    auto kern = fp8_gemm_small_tile_kernel<TILE, STAGES, EDGE, false>;
    constexpr int lds_bytes = STAGES * 2 * TILE * BK;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + TILE - 1) / TILE, tiles_n = (N + TILE - 1) / TILE;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream,
                       (const uint8_t*)A, (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha, tiles_m,
                       tiles_n, 0, (float*)nullptr);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <bool EDGE>
static int launch_tile128_splitk(const void* A, const void* B, void* C, int M, int N, int K, float alpha,
                                 int splits, float* partial, hipStream_t stream) {
    static DeviceOnce configured;
    return launch_small_tile_splitk(fp8_gemm_small_tile_kernel<kTinyTile, kTinyStages, EDGE, true>, configured, A,
                                    B, C, M, N, K, alpha, splits, partial, stream);
}

template <bool EDGE>
static int launch_4wave(const void* A, const void* B, void* C, int M, int N, int K, float alpha,
                        hipStream_t stream) {
    auto kern = fp8_gemm_4wave_ring_kernel<EDGE>;
    constexpr int lds_bytes = 5 * kTileBytes;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream,
                       (const uint8_t*)A, (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha, tiles_m,
                       tiles_n, raster_band(((long long)M + N) * K, tiles_n));
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

}  // namespace hk

extern "C" int hk_fp8_gemm_variant(const void* A, const void* B, void* C, int M, int N, int K,
                                   float scale_a, float scale_b, int variant, void* stream) {
    using namespace hk;
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 16) != 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (variant < 0 || variant > 8 || variant == 2 || variant == 3) return HK_ERR_UNSUPPORTED;
    if (variant == 8 && M > kSkinnyMaxM) return HK_ERR_UNSUPPORTED;
    // K tails: the tile kernels zero-fill the last K-step of any K % 16 == 0
    if (variant != 0 && (long long)K * BM >= (1ll << 31)) return HK_ERR_BAD_SHAPE;
    const float alpha = scale_a * scale_b;
    hipStream_t s = (hipStream_t)stream;
    if (variant == 0) {
        if ((long long)((M + 63) / 64) > 65535) return HK_ERR_BAD_SHAPE;
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        hipLaunchKernelGGL(fp8_gemm_portable_kernel, grid, dim3(256), 0, s, (const uint8_t*)A,
                           (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha);
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    if (variant == 5) {
        const bool edge128 = (M % kSmallTile) != 0 || (N % kSmallTile) != 0;
        return edge128 ? launch_small_tile<kSmallTile, kSmallStages, true>(A, B, C, M, N, K, alpha, s)
                       : launch_small_tile<kSmallTile, kSmallStages, false>(A, B, C, M, N, K, alpha, s);
    }
    if (variant == 6) {
        const bool edge64 = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
        return edge64 ? launch_small_tile<kTinyTile, kTinyStages, true>(A, B, C, M, N, K, alpha, s)
                      : launch_small_tile<kTinyTile, kTinyStages, false>(A, B, C, M, N, K, alpha, s);
    }
    if (variant == 8) return launch_skinny(A, B, C, M, N, K, alpha, s);
    if (variant == 7) {
        const bool e = (M % kPcBM) != 0 || (N % BN) != 0;
        return e ? launch_prodcons<true>(A, B, C, M, N, K, alpha, s) : launch_prodcons<false>(A, B, C, M, N, K, alpha, s);
    }
    const bool edge = (M % BM) != 0 || (N % BN) != 0;
    if (variant == 1)
        return edge ? launch_pingpong<true>(A, B, C, M, N, K, alpha, s) : launch_pingpong<false>(A, B, C, M, N, K, alpha, s);
    return edge ? launch_4wave<true>(A, B, C, M, N, K, alpha, s) : launch_4wave<false>(A, B, C, M, N, K, alpha, s);
}

extern "C" size_t hk_fp8_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || hk::gemm_dims_too_large(M, N, K)) return 0;
    const int s = hk::splitk_ranges(M, N, K);
    return s < 2 ? 0 : (size_t)s * M * N * sizeof(float);
}

extern "C" int hk_fp8_gemm_ws(const void* A, const void* B, void* C, int M, int N, int K, float scale_a,
                              float scale_b, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const int splits = splitk_ranges(M, N, K);
    const bool can_split = splits >= 2 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) &&
                           (K % 16) == 0 && (long long)K * BM < (1ll << 31) && (long long)M * N < (1ll << 40);
    if (!can_split) return hk_fp8_gemm(A, B, C, M, N, K, scale_a, scale_b, stream);
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)workspace) & 15u) return HK_ERR_BAD_ALIGNMENT;
    // the skinny kernel adds its partial sums inside the workgroup and leaves the workspace alone
    if (use_skinny(M, N, (K + BK - 1) / BK, true, moe_num_compute_units()))
        return hk_fp8_gemm_variant(A, B, C, M, N, K, scale_a, scale_b, 8, stream);
    const bool edge = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
    const float alpha = scale_a * scale_b;
    return edge ? launch_tile128_splitk<true>(A, B, C, M, N, K, alpha, splits, (float*)workspace, (hipStream_t)stream)
                : launch_tile128_splitk<false>(A, B, C, M, N, K, alpha, splits, (float*)workspace, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------
// Split-K partial sums in device memory that belongs to the library: a file-scope array that every
// GPU the library is loaded on holds from then until the process ends. 8 MiB covers every shape the
// split-K path takes on a 256-CU device (ranges x 64x64 tiles <= 512 workgroups, 16 KiB of fp32
// partial sums each).
namespace hk {
constexpr size_t kStaticScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// The array's address on each device (every GPU has its own copy at its own address), looked up
// once per device with that device current. Host code uses these pointers, never the array's name.
static std::atomic<void*> scratch_ptr[64];

static int static_scratch(void** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return HK_ERR_LAUNCH;
    if (dev < 0 || dev >= 64) return HK_ERR_UNSUPPORTED;   // (the caller then runs without a split)
    void* p = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return HK_ERR_LAUNCH;
        scratch_ptr[dev].store(p, std::memory_order_release);   // a racing thread stores the same address
    }
    *out = p;
    return HK_OK;
}
}  // namespace hk

extern "C" size_t hk_fp8_gemm_static_ws_max_bytes(void) { return hk::kStaticScratchBytes; }

extern "C" int hk_fp8_gemm_static_ws(const void* A, const void* B, void* C, int M, int N, int K, float scale_a,
                                     float scale_b, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const int splits = splitk_ranges(M, N, K);
    if (splits < 2) return hk_fp8_gemm(A, B, C, M, N, K, scale_a, scale_b, stream);   // no scratch needed
    // splitk_ranges gives at most two workgroups per CU, 16 KiB of partial sums each: the array covers devices
    // of up to 256 CUs; a larger device can ask for more, which is refused (the caller then uses hk_fp8_gemm_ws
    // or hk_fp8_gemm)
    static_assert(kStaticScratchBytes == (size_t)2 * 256 * kTinyTile * kTinyTile * sizeof(float), "512 workgroups' partial sums");
    const size_t need = (size_t)splits * M * N * sizeof(float);
    if (need > kStaticScratchBytes) return HK_ERR_WORKSPACE;   // more partial sums than the array holds
    void* ws = nullptr;
    const int st = static_scratch(&ws);
    // a device ordinal this table does not cover: the same result without a split, as hk_fp8_gemm_ws does
    // without a workspace
    if (st == HK_ERR_UNSUPPORTED) return hk_fp8_gemm(A, B, C, M, N, K, scale_a, scale_b, stream);
    if (st != HK_OK) return st;
    // every partial sum that the reduction reads is written by this call's first kernel: nothing in
    // the array needs clearing between calls
    return hk_fp8_gemm_ws(A, B, C, M, N, K, scale_a, scale_b, ws, kStaticScratchBytes, stream);
}

extern "C" int hk_gemm_tile_choice(int format, int M, int N, int K, int consult_table) {
    using namespace hk;
    if (format < 0 || format > 2 || M <= 0 || N <= 0 || K <= 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const long long row_bytes = format == kFmtFp8 ? K : format == kFmtBf16 ? 2ll * K : K / 2;
    const int nk = (int)((row_bytes + BK - 1) / BK);
    const TileRule rule = format == kFmtFp8 ? kTileRuleFp8 : format == kFmtBf16 ? kTileRuleBf16 : kTileRuleMxfp4;
    return pick_tile(format, M, N, nk, rule, consult_table != 0);
}

extern "C" int hk_fp8_gemm(const void* A, const void* B, void* C, int M, int N, int K,
                           float scale_a, float scale_b, void* stream) {
    using namespace hk;
    if (gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const bool tile_ok = K > 0 && (long long)K * BM < (1ll << 31);
    // 256x256 tiles (five-slot ring kernel), 128x128 or 64x64: see pick_tile
    const int tile = pick_tile(kFmtFp8, M, N, (K + BK - 1) / BK, kTileRuleFp8);
    // few rows: one pass over B by the skinny kernel where that is faster (use_skinny)
    const bool skinny = tile_ok && use_skinny(M, N, (K + BK - 1) / BK, false, moe_num_compute_units());
    const int variant = !tile_ok ? 0 : skinny ? 8 : tile == kTinyTile ? 6 : tile == kSmallTile ? 5 : 4;
    return hk_fp8_gemm_variant(A, B, C, M, N, K, scale_a, scale_b, variant, stream);
}
