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
#include "gemm_small_tile.h"
#include "gemm_pingpong.h"
#include "../../include/hk355.h"

namespace hk {

// ---------------------------------------------------------------------------------------
// 4-wave kernel with a five-slot LDS ring (all 160 KiB): two slots for A tiles, three for B
// tiles. One wave per SIMD, each owning a 128x128 patch of the 256x256 tile (8x8 MFMA tiles, 256
// accumulator registers); every LDS read, global->LDS load and MFMA has a fixed place in the
// instruction stream (one MFMA per "slot", memory operations attached to slots): A fragment m + 3 is
// read while the MFMAs of fragment m issue, the next K-step's B fragments after the single barrier per
// K-step (schedule idea after the reference's 4-wave kernel, kernels/gemm/fp8fp32/README.md:3-5,
// per-instruction helpers in FP8_4wave/utils.cpp:44-52, 131-137, 150-161). The global->LDS loads are
// spread over the whole K-step instead of being bunched behind the barrier: the address unit of a CU
// needs 16 cycles per 1 KiB load, 16 loads per wave and step, and a wave that cannot hand
// its load over also cannot issue its next MFMA. B fragments of tile kt are read one step
// early (after barrier kt-1), so with a third B slot tile kt+2 of B may be fetched during
// MFMA groups 0..PG of step kt; A tile kt+2 follows after the barrier into the A slot that
// step kt has just finished reading.
template <bool EDGE>
__global__ __launch_bounds__(256) void fp8_gemm_4wave_ring_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n) {
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
        banded_raster(id, tiles_m, tiles_n, 4, band_n, pm, pn);
    }
    const int row0 = pm * BM, col0 = pn * BN;

    const int a_rows = min(M - row0, BM), b_rows = min(N - col0, BN);
    const v4i srd_a = make_srd(A + (size_t)row0 * K, (uint32_t)a_rows * (uint32_t)K);
    const v4i srd_b = make_srd(B + (size_t)col0 * K, (uint32_t)b_rows * (uint32_t)K);

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
        voff_a[i] = (uint32_t)ra * (uint32_t)K + c * 16u;
        voff_b[i] = (uint32_t)rb * (uint32_t)K + c * 16u;
    }
    const uint32_t dma_row_stride = to_sgpr((uint32_t)(8 * NW) * (uint32_t)K);
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
    v8i bf[2][NT];  // B fragments of the current / next K-step
    v8i af[4];      // rotating A fragments

    const int nk = (K + BK - 1) / BK;
    // the chunk a lane fetches is the same for all of its loads: swz(row, lane % 8) with row bits
    // [1..3] = 4 w + lane / 16 (mod 8)
    const uint32_t tail_or =
        (int)(swz_chunk(8 * w + (lane >> 3), lane & 7) * 16u) >= K - (nk - 1) * BK ? 0x80000000u : 0u;

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
    for (int n = 0; n < NT; ++n) bf[0][n] = lds_frag(b_lo0, b_hi0, n * 16 * BK);
#pragma unroll
    for (int m = 0; m < AD; ++m) af[m] = lds_frag(a_lo[0], a_hi[0], m * 16 * BK);

    // B ring positions (byte offsets): tile kt+1 is read from off1, tile kt+2 is loaded to off2.
    uint32_t off1 = kTileBytes, off2 = 2 * kTileBytes;

    // One K-step with A slot / fragment parity P. Every step runs the same code: the last step's
    // prefetch reads return stale LDS contents that are never used, and refills past the end of K
    // are issued against a zero-sized buffer (out of range for every lane, no memory traffic), so
    // that no step needs a differently scheduled body.
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
                mfma_fp8_16x16x128_acc(acc[m][n], bf[P][n], af[m & 3]);
                if (m <= PG) {
                    const int s = m * NT + n;  // 40 slots before the barrier: B loads at 2, 7, .., 37
                    if (n == 0) af[(m + AD) & 3] = lds_frag(a_lo[P], a_hi[P], (m + AD) * 16 * BK);
                    if (s % 5 == 2) dma_b(s / 5, off2, k2, sb, vor);
                } else {
                    const int j = (m - PG - 1) * NT + n;  // 24 slots after the barrier
                    if (j < NT) {
                        bf[P ^ 1][j] = lds_frag(bl, bh, j * 16 * BK);
                    } else if (j == NT || j == NT + 1) {
                        af[j - NT] = lds_frag(a_lo[P ^ 1], a_hi[P ^ 1], (j - NT) * 16 * BK);
                    } else if (j == 2 * NT) {
                        af[2] = lds_frag(a_lo[P ^ 1], a_hi[P ^ 1], 2 * 16 * BK);
                    }
                    if (j < 2 * NDMA && (j & 1)) dma_a(j >> 1, P, k2, sa, vor);  // A loads at 1, 3, .., 15
                }
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
    if (M <= 0 || N <= 0 || K <= 0 || (K % 16) != 0) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (variant < 0 || variant > 6 || variant == 2 || variant == 3) return HK_ERR_UNSUPPORTED;
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
    const bool edge = (M % BM) != 0 || (N % BN) != 0;
    if (variant == 1)
        return edge ? launch_pingpong<true>(A, B, C, M, N, K, alpha, s) : launch_pingpong<false>(A, B, C, M, N, K, alpha, s);
    return edge ? launch_4wave<true>(A, B, C, M, N, K, alpha, s) : launch_4wave<false>(A, B, C, M, N, K, alpha, s);
}

extern "C" size_t hk_fp8_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const int s = hk::splitk_ranges(M, N, K);
    return s < 2 ? 0 : (size_t)s * M * N * sizeof(float);
}

extern "C" int hk_fp8_gemm_ws(const void* A, const void* B, void* C, int M, int N, int K, float scale_a,
                              float scale_b, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0) return HK_ERR_BAD_SHAPE;
    const int splits = splitk_ranges(M, N, K);
    const bool can_split = splits >= 2 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) &&
                           (K % 16) == 0 && (long long)K * BM < (1ll << 31) && (long long)M * N < (1ll << 40);
    if (!can_split) return hk_fp8_gemm(A, B, C, M, N, K, scale_a, scale_b, stream);
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)workspace) & 15u) return HK_ERR_BAD_ALIGNMENT;
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
    if (dev < 0 || dev >= 64) return HK_ERR_UNSUPPORTED;
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
    if (M <= 0 || N <= 0 || K <= 0) return HK_ERR_BAD_SHAPE;
    const int splits = splitk_ranges(M, N, K);
    if (splits < 2) return hk_fp8_gemm(A, B, C, M, N, K, scale_a, scale_b, stream);   // no scratch needed
    const size_t need = (size_t)splits * M * N * sizeof(float);
    if (need > kStaticScratchBytes) return HK_ERR_WORKSPACE;   // more partial sums than the array holds
    void* ws = nullptr;
    const int st = static_scratch(&ws);
    if (st != HK_OK) return st;
    // every partial sum that the reduction reads is written by this call's first kernel: nothing in
    // the array needs clearing between calls
    return hk_fp8_gemm_ws(A, B, C, M, N, K, scale_a, scale_b, ws, kStaticScratchBytes, stream);
}

extern "C" int hk_fp8_gemm(const void* A, const void* B, void* C, int M, int N, int K,
                           float scale_a, float scale_b, void* stream) {
    using namespace hk;
    const bool tile_ok = K > 0 && (long long)K * BM < (1ll << 31);
    // The tile is the largest that still gives every CU of an MI355X work: 256x256 (five-slot ring
    // kernel) from 128 such tiles on; below that 128x128 tiles, and 64x64 tiles (two workgroups
    // per CU) when even those number at most 128.
    const long long tiles256 = (long long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    const long long tiles128 =
        (long long)((M + kSmallTile - 1) / kSmallTile) * ((N + kSmallTile - 1) / kSmallTile);
    const int variant = !tile_ok ? 0 : tiles128 <= 128 ? 6 : tiles256 < 128 ? 5 : 4;
    return hk_fp8_gemm_variant(A, B, C, M, N, K, scale_a, scale_b, variant, stream);
}
