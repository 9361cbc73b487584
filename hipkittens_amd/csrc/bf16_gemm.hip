// BF16 GEMM for gfx950: C[M,N] = bf16( A[M,K] * B[N,K]^T ), bf16 operands, fp32 accumulate.
//
// Counterpart of the reference's flagship kernel (kernels/gemm/bf16fp32/mi350x, bound as
// tk_kernel.dispatch_micro(A, B, C), kernels/gemm/bf16fp32/mi350x/test_python.py:80-82; tile
// 256x256x64, kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:13-42), built on this library's FP8
// skeleton to show that the schedule is independent of the operand type: a K-step is again
// 128 bytes per operand row (64 bf16 elements), so tile layout, swizzle, direct global->LDS
// loads, the five-slot LDS ring and the slot plan are those of fp8_gemm_4wave_ring_kernel; the
// two 16-byte halves a lane reads per fragment row are K elements 8g.. and 32 + 8g.. and feed
// two v_mfma_f32_16x16x32_bf16 (16 cycles each, together as long as one FP8 MFMA).
#include "gemm_tile.h"
#include "gemm_small_tile.h"
#include "gemm_pingpong.h"
#include "../../include/hk355.h"

namespace hk {

// acc(16x16) += X(16x32 bf16) * Y(16x32 bf16)^T with the accumulator tied in place in an AGPR;
// lane l supplies row l % 16, K elements 8 (l / 16) .. +8 of each operand.
__device__ __forceinline__ void mfma_bf16_16x16x32_acc(v4f& acc, const v4i& x, const v4i& y) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
}

// See fp8_gemm_4wave_ring_kernel (fp8_gemm.hip) for the ring, the slot plan and the uniform tail.
template <bool EDGE>
__global__ __launch_bounds__(256) void bf16_gemm_4wave_ring_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
    const int Kb = 2 * K;  // operand row pitch in bytes; a K-step is 128 bytes = 64 elements
    constexpr int NW = 4, TM = 128, TN = 128, MT = 8, NT = 8;
    constexpr int NDMA = kTileBytes / (NW * 1024);  // 8 loads per wave per operand per K-step
    constexpr int PG = 4, AD = 3;
    constexpr uint32_t kBRing = 2 * kTileBytes;      // B slots start behind the two A slots
    static_assert(PG == 4 && AD == 3 && MT == 8 && NDMA == 8, "slot plan below is written for these");
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];

    const int lane = lane_id();
    const int w = wave_id();
    const int wm = w >> 1, wn = w & 1;

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        banded_raster(id, tiles_m, tiles_n, band_n < tiles_n ? 4 : 8, band_n, pm, pn);
    }
    const int row0 = pm * BM, col0 = pn * BN;

    const int a_rows = min(M - row0, BM), b_rows = min(N - col0, BN);
    const v4i srd_a = make_srd(A + (size_t)row0 * Kb, (uint32_t)a_rows * (uint32_t)Kb);
    const v4i srd_b = make_srd(B + (size_t)col0 * Kb, (uint32_t)b_rows * (uint32_t)Kb);

    uint32_t voff_a[EDGE ? NDMA : 1], voff_b[EDGE ? NDMA : 1];
#pragma unroll
    for (int i = 0; i < (EDGE ? NDMA : 1); ++i) {
        const int R = 8 * (i * NW + w) + (lane >> 3);
        const uint32_t c = swz_chunk(R, lane & 7);
        int ra = R, rb = b_row_to_col(R);
        if (EDGE) {
            ra = min(ra, a_rows - 1);
            rb = min(rb, b_rows - 1);
        }
        voff_a[i] = (uint32_t)ra * (uint32_t)Kb + c * 16u;
        voff_b[i] = (uint32_t)rb * (uint32_t)Kb + c * 16u;
    }
    const uint32_t dma_row_stride = to_sgpr((uint32_t)(8 * NW) * (uint32_t)Kb);
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);

    // One global->LDS load of A (into A slot `slot`) or B (into the B slot at byte offset
    // `slot_off` of the B ring).
    // `vor` is 0, or for the last K-step of a K that is not a multiple of the K-step the lane's
    // tail_or: bit 31 moves the lanes whose 16-byte chunk lies past the end of the row out of the
    // buffer's range, and such lanes write zeros to LDS.
    auto dma_a = [&](int i, int slot, uint32_t k0, v4i srd, uint32_t vor) {
        const uint32_t dst = lds_wave + (uint32_t)slot * kTileBytes + i * NW * 1024;
        if (EDGE)
            dma16(srd, dst, voff_a[i] | vor, k0);
        else
            dma16(srd, dst, voff_a[0] | vor, k0 + i * dma_row_stride);
    };
    auto dma_b = [&](int i, uint32_t slot_off, uint32_t k0, v4i srd, uint32_t vor) {
        const uint32_t dst = lds_wave + kBRing + slot_off + i * NW * 1024;
        if (EDGE)
            dma16(srd, dst, voff_b[i] | vor, k0);
        else
            dma16(srd, dst, voff_b[0] | vor, k0 + i * dma_row_stride);
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    uint32_t a_lo[2], a_hi[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
        a_lo[st] = lds0 + st * kTileBytes + wm * (TM * BK) + rd_lo;
        a_hi[st] = lds0 + st * kTileBytes + wm * (TM * BK) + rd_hi;
    }
    const uint32_t b_lo0 = lds0 + kBRing + wn * (TN * BK) + rd_lo;
    const uint32_t b_hi0 = lds0 + kBRing + wn * (TN * BK) + rd_hi;

    v4f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
    Frag4 bf[2][NT];  // B fragments of the current / next K-step (lo: K 0..31, hi: K 32..63)
    Frag4 af[4];      // rotating A fragments

    const int nk = (Kb + BK - 1) / BK;
    // the chunk a lane fetches is the same for all of its loads: swz(row, lane % 8) with row bits
    // [1..3] = 4 w + lane / 16 (mod 8)
    const uint32_t tail_or =
        (int)(swz_chunk(8 * w + (lane >> 3), lane & 7) * 16u) >= Kb - (nk - 1) * BK ? 0x80000000u : 0u;

    // ---- prologue: tiles 0 and 1 in flight, first fragments in registers ------------------
    {
        const uint32_t vor = nk == 1 ? tail_or : 0u;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_b(i, 0, 0, srd_b, vor);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_a(i, 0, 0, srd_a, vor);
    }
    wait_vmcnt<0>();
    block_barrier();
    {
        v4i sa = srd_a, sb = srd_b;
        if (nk < 2) { sa.z = 0; sb.z = 0; }
        const uint32_t vor = nk == 2 ? tail_or : 0u;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_b(i, kTileBytes, BK, sb, vor);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_a(i, 1, BK, sa, vor);
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) bf[0][n] = lds_frag4(b_lo0, b_hi0, n * 16 * BK);
#pragma unroll
    for (int m = 0; m < AD; ++m) af[m] = lds_frag4(a_lo[0], a_hi[0], m * 16 * BK);

    // B ring positions (byte offsets): tile kt+1 is read from off1, tile kt+2 is loaded to off2.
    uint32_t off1 = kTileBytes, off2 = 2 * kTileBytes;

    // One K-step with A slot / fragment parity P. Every step runs the same code (refills past the end
    // of K go against a zero-sized buffer, the last step's prefetch reads are never used: see
    // fp8_gemm_4wave_ring_kernel).
    auto step = [&]<int P>(int kt) {
        const uint32_t k2 = (uint32_t)(kt + 2) * BK;
        v4i sa = srd_a, sb = srd_b;
        if (kt + 2 >= nk) { sa.z = 0; sb.z = 0; }
        const uint32_t vor = kt + 2 == nk - 1 ? tail_or : 0u;
        const uint32_t bl = b_lo0 + off1, bh = b_hi0 + off1;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                mfma_bf16_16x16x32_acc(acc[m][n], bf[P][n].lo, af[m & 3].lo);
                if (m <= PG) {
                    const int s = m * NT + n;  // 40 slots before the barrier: B loads at 2, 7, .., 37
                    if (n == 0) af[(m + AD) & 3] = lds_frag4(a_lo[P], a_hi[P], (m + AD) * 16 * BK);
                    if (s % 5 == 2) dma_b(s / 5, off2, k2, sb, vor);
                } else {
                    const int j = (m - PG - 1) * NT + n;  // 24 slots after the barrier
                    if (j < NT) {
                        bf[P ^ 1][j] = lds_frag4(bl, bh, j * 16 * BK);
                    } else if (j == NT || j == NT + 1) {
                        af[j - NT] = lds_frag4(a_lo[P ^ 1], a_hi[P ^ 1], (j - NT) * 16 * BK);
                    } else if (j == 2 * NT) {
                        af[2] = lds_frag4(a_lo[P ^ 1], a_hi[P ^ 1], 2 * 16 * BK);
                    }
                    if (j < 2 * NDMA && (j & 1)) dma_a(j >> 1, P, k2, sa, vor);  // A loads at 1, 3, .., 15
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // second half of the K-step on the same fragments; the two MFMAs into one
            // accumulator are 8 issue slots apart
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                mfma_bf16_16x16x32_acc(acc[m][n], bf[P][n].hi, af[m & 3].hi);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG) {
                // every read of A slot P by this wave has been issued; tile kt+1 (all loads
                // but the 8 B loads of this step) must have landed for all waves
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                wait_vmcnt<NDMA>();
                block_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        off1 = off2;
        off2 = off2 == 2 * kTileBytes ? 0u : off2 + kTileBytes;
    };

    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        step.template operator()<0>(kt);
        step.template operator()<1>(kt + 1);
    }
    if (kt < nk) step.template operator()<0>(kt);
    wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup retires
    mfma_drain_agpr(acc);

    store_c_tile<MT, NT, EDGE>(acc, C, M, N, row0 + wm * TM, col0 + wn * TN, alpha);
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

template <bool EDGE>
static int launch_bf16_ring(const void* A, const void* B, void* C, int M, int N, int K, hipStream_t stream) {
    auto kern = bf16_gemm_4wave_ring_kernel<EDGE>;
    constexpr int lds_bytes = 5 * kTileBytes;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)B, (uint16_t*)C, M, N, K, 1.0f, tiles_m, tiles_n,
                       raster_band(((long long)M + N) * K * 2, tiles_n));
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

}  // namespace hk

extern "C" int hk_bf16_gemm_variant(const void* A, const void* B, void* C, int M, int N, int K, int variant,
                                    void* stream) {
    using namespace hk;
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 8) != 0) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (variant < 0 || variant > 4) return HK_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (variant == 0) {
        if ((long long)((M + 63) / 64) > 65535) return HK_ERR_BAD_SHAPE;
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        hipLaunchKernelGGL(bf16_gemm_portable_kernel, grid, dim3(256), 0, s, (const uint16_t*)A,
                           (const uint16_t*)B, (uint16_t*)C, M, N, K, 1.0f);
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    if ((long long)2 * K * BM >= (1ll << 31)) return HK_ERR_BAD_SHAPE;
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
    const bool edge = (M % BM) != 0 || (N % BN) != 0;
    if (variant == 4)
        return edge ? launch_bf16_pingpong<true>(A, B, C, M, N, K, s) : launch_bf16_pingpong<false>(A, B, C, M, N, K, s);
    return edge ? launch_bf16_ring<true>(A, B, C, M, N, K, s) : launch_bf16_ring<false>(A, B, C, M, N, K, s);
}

extern "C" int hk_bf16_gemm(const void* A, const void* B, void* C, int M, int N, int K, void* stream) {
    using namespace hk;
    const bool tile_ok = K > 0 && (long long)2 * K * BM < (1ll << 31);
    // the same choice of tile as hk_fp8_gemm: the largest that still gives every CU work
    const long long tiles256 = (long long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    const long long tiles128 =
        (long long)((M + kSmallTile - 1) / kSmallTile) * ((N + kSmallTile - 1) / kSmallTile);
    const int variant = !tile_ok ? 0 : tiles128 <= 128 ? 3 : tiles256 < 128 ? 2 : 1;
    return hk_bf16_gemm_variant(A, B, C, M, N, K, variant, stream);
}

extern "C" size_t hk_bf16_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || K >= (1 << 30)) return 0;
    const int s = hk::splitk_ranges(M, N, 2 * K);
    return s < 2 ? 0 : (size_t)s * M * N * sizeof(float);
}

extern "C" int hk_bf16_gemm_ws(const void* A, const void* B, void* C, int M, int N, int K, void* workspace,
                               size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0) return HK_ERR_BAD_SHAPE;
    const int splits = K < (1 << 30) ? splitk_ranges(M, N, 2 * K) : 1;
    const bool can_split = splits >= 2 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) &&
                           (K % 8) == 0 && (long long)2 * K * BM < (1ll << 31) && (long long)M * N < (1ll << 40);
    if (!can_split) return hk_bf16_gemm(A, B, C, M, N, K, stream);
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)workspace) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const bool edge = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
    return edge ? launch_bf16_splitk<true>(A, B, C, M, N, K, splits, (float*)workspace, (hipStream_t)stream)
                : launch_bf16_splitk<false>(A, B, C, M, N, K, splits, (float*)workspace, (hipStream_t)stream);
}
