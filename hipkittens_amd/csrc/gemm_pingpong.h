// 8-wave ping-pong GEMM body for the 256x256 tile, shared by the FP8, BF16 and MXFP4 GEMMs (a K-step
// is 128 bytes per operand row in all three; only the MFMA differs).
//
// The schedule follows the reference's flagship kernel (kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:
// 73-77 the extra barrier that offsets the second wave group, 88-153 the alternating memory / MFMA
// clusters, 219-221 the matching barrier at the end; kernels/gemm/fp8fp32/README.md:3-5 names it as the
// second FP8 schedule): two groups of four waves, one wave of each group per SIMD. A K-step is four phases,
//   P0 memory : global->LDS loads of the next tile, LDS reads of this tile's B fragments and of the
//               first half of the wave's A fragments
//   P1 MFMA   : the 16 MFMA tiles of the first half (raised priority)
//   P2 memory : LDS reads of the second half of the A fragments; the wave's loads must have landed
//   P3 MFMA   : the 16 MFMA tiles of the second half
// each closed by a workgroup barrier. The second group runs one phase behind the first (it passes one
// barrier more before its first phase and the first group one more at the end), so while one wave of a
// SIMD issues MFMAs the other reads LDS, issues loads or waits at its s_waitcnt. That is what a single
// wave per SIMD cannot do for the 16-cycle MFMAs (BF16, FP4), which leave three issue slots between
// two MFMAs.
// Tile format, swizzle, B-row permutation, K tail and epilogue are those of the other tile kernels
// (gemm_tile.h); wave (wm, wn) owns rows [64 wm, +64) and [128 + 64 wm, +64) x columns [64 wn, +64) of
// the tile. Two LDS stages: the next tile is loaded while this one is multiplied. Every output
// element sums its K-steps in the same order as in the other tile kernels: identical bits.
#pragma once
#include "gemm_small_tile.h"

namespace hk {

constexpr int kPpScaleSlot = 2 * BM * 16;                       // MXFP4: 16 scale bytes (two K-steps) per row of A, then of B
constexpr int kPpLdsBytes = kLdsBytes;                          // two stages of A tile + B tile (128 KiB)
constexpr int kPpLdsBytesScaled = kLdsBytes + 2 * kPpScaleSlot; // + two scale slots (16 KiB)

// MMA: as in gemm_small_tile_body (MMA::kScaled: MXFP4 with e8m0 scales, rows of sa_pitch / sb_pitch bytes).
// K: the operands' row length in BYTES (a multiple of 16).
template <typename MMA, bool EDGE>
__device__ __forceinline__ void gemm_pingpong_body(
    uint8_t* smem, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int band_n,
    SmallTileScales sc = SmallTileScales{nullptr, nullptr, 0, 0}) {
    constexpr int NW = 8, HM = 4, NT = 4;            // per wave: two halves of HM x NT MFMA tiles
    constexpr int NDMA = kTileBytes / (NW * 1024);   // 4 loads per wave per operand per K-step
    constexpr bool kScaled = MMA::kScaled;
    const int lane = lane_id(), w = wave_id();
    const int wm = w >> 2, wn = w & 3;

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        banded_raster(id, tiles_m, tiles_n, band_n < tiles_n ? 4 : 8, band_n, pm, pn);
    }
    const int row0 = pm * BM, col0 = pn * BN;
    const int a_rows = min(M - row0, BM), b_rows = min(N - col0, BN);
    const v4i srd_a = make_srd(A + (size_t)row0 * K, (uint32_t)a_rows * (uint32_t)K);
    const v4i srd_b = make_srd(B + (size_t)col0 * K, (uint32_t)b_rows * (uint32_t)K);

    uint32_t voff_a[NDMA], voff_b[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
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
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const int nk = (K + BK - 1) / BK;
    // last K-step of a K that is not a multiple of 128: lanes whose 16-byte chunk lies past the end of
    // the row are moved out of the buffer's range (bit 31) and write zeros to LDS. The chunk a lane
    // fetches is the same for all of its loads: swz(row, lane % 8) with row bits [1..3] = 4 w + lane / 16 (mod 8)
    const uint32_t tail_or =
        (int)(swz_chunk(8 * w + (lane >> 3), lane & 7) * 16u) >= K - (nk - 1) * BK ? 0x80000000u : 0u;
    // Scale loads (kScaled): wave w fetches operand w & 1 (0 = A), lane l the 16 bytes of row 64 (w >> 1) + l,
    // i.e. the scales of the pair of K-steps kt / 2, with every K-step (on odd K-steps it repeats the pair's
    // load into the same slot, which keeps the number of loads per K-step uniform).
    v4i srd_s = {0, 0, 0, 0};
    uint32_t voff_s = 0, lds_s = 0;
    if (kScaled) {
        const int op = w & 1, srow0 = 64 * (w >> 1);
        const int R = srow0 + lane;
        int rr = op ? b_row_to_col(R) : R;
        if (EDGE) rr = min(rr, (op ? b_rows : a_rows) - 1);
        const int pitch = op ? sc.sb_pitch : sc.sa_pitch;
        srd_s = op ? make_srd(sc.SB + (size_t)col0 * pitch, (uint32_t)b_rows * (uint32_t)pitch)
                   : make_srd(sc.SA + (size_t)row0 * pitch, (uint32_t)a_rows * (uint32_t)pitch);
        voff_s = (uint32_t)rr * (uint32_t)pitch;
        lds_s = to_sgpr(lds0 + kPpLdsBytes + (uint32_t)op * (BM * 16) + (uint32_t)srow0 * 16u);
    }
    auto issue_tile = [&](int kt) {
        const uint32_t k0 = (uint32_t)kt * BK;
        const uint32_t dst = lds_wave + (uint32_t)(kt & 1) * kStageBytes;
        const uint32_t vor = kt == nk - 1 ? tail_or : 0u;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma16(srd_a, dst + i * NW * 1024, voff_a[i] | vor, k0);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma16(srd_b, dst + kTileBytes + i * NW * 1024, voff_b[i] | vor, k0);
        if (kScaled) dma16(srd_s, lds_s + (uint32_t)((kt >> 1) & 1) * kPpScaleSlot, voff_s, (uint32_t)(kt >> 1) * 16u);
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    // A fragments of half h: tile rows 128 h + 64 wm + 16 m + r
    const uint32_t a_lo0 = lds0 + wm * (64 * BK) + rd_lo, a_hi0 = lds0 + wm * (64 * BK) + rd_hi;
    const uint32_t b_lo0 = lds0 + kTileBytes + wn * (64 * BK) + rd_lo;
    const uint32_t b_hi0 = lds0 + kTileBytes + wn * (64 * BK) + rd_hi;

    v4f acc[2][HM][NT];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int m = 0; m < HM; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[h][m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    issue_tile(0);
    wait_vmcnt<0>();
    block_barrier();
    if (wm == 1) block_barrier();   // the second group runs one phase behind the first

    for (int kt = 0; kt < nk; ++kt) {
        const uint32_t so = (uint32_t)(kt & 1) * kStageBytes;
        // ---- P0 memory ---------------------------------------------------------------------
        if (kt + 1 < nk) issue_tile(kt + 1);
        v8i bf[NT], af[HM];
        v2i bs[NT], as[HM];
        uint32_t sbase = 0;
        const uint32_t sh = 8u * g;
#pragma unroll
        for (int n = 0; n < NT; ++n) bf[n] = lds_frag(b_lo0 + so, b_hi0 + so, n * 16 * BK);
#pragma unroll
        for (int m = 0; m < HM; ++m) af[m] = lds_frag(a_lo0 + so, a_hi0 + so, m * 16 * BK);
        if constexpr (kScaled) {
            // the lane's scale bytes: row 16 f + r of the wave's patch, byte g of each K half's dword
            sbase = lds0 + kPpLdsBytes + (uint32_t)((kt >> 1) & 1) * kPpScaleSlot + (uint32_t)(kt & 1) * 8u + r * 16u;
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                bs[n] = *(lds_v2i_t*)(uintptr_t)(sbase + BM * 16 + (wn * 64 + 16 * n) * 16);
                bs[n].x = (int)((uint32_t)bs[n].x >> sh); bs[n].y = (int)((uint32_t)bs[n].y >> sh);
            }
#pragma unroll
            for (int m = 0; m < HM; ++m) {
                as[m] = *(lds_v2i_t*)(uintptr_t)(sbase + (wm * 64 + 16 * m) * 16);
                as[m].x = (int)((uint32_t)as[m].x >> sh); as[m].y = (int)((uint32_t)as[m].y >> sh);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- P1 MFMA -----------------------------------------------------------------------
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int m = 0; m < HM; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                if constexpr (kScaled) MMA::mma(acc[0][m][n], bf[n], af[m], bs[n], as[m]);
                else MMA::mma(acc[0][m][n], bf[n], af[m]);
            }
        __builtin_amdgcn_s_setprio(0);
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- P2 memory ---------------------------------------------------------------------
#pragma unroll
        for (int m = 0; m < HM; ++m) af[m] = lds_frag(a_lo0 + so, a_hi0 + so, (128 + m * 16) * BK);
        if constexpr (kScaled) {
#pragma unroll
            for (int m = 0; m < HM; ++m) {
                as[m] = *(lds_v2i_t*)(uintptr_t)(sbase + (128 + wm * 64 + 16 * m) * 16);
                as[m].x = (int)((uint32_t)as[m].x >> sh); as[m].y = (int)((uint32_t)as[m].y >> sh);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait_vmcnt<0>();   // this wave's part of the next tile has landed (everyone's: after the barrier behind the second group's P2)
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- P3 MFMA -----------------------------------------------------------------------
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int m = 0; m < HM; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                if constexpr (kScaled) MMA::mma(acc[1][m][n], bf[n], af[m], bs[n], as[m]);
                else MMA::mma(acc[1][m][n], bf[n], af[m]);
            }
        __builtin_amdgcn_s_setprio(0);
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    if (wm == 0) block_barrier();   // matches the second group's extra barrier at the start

    store_c_tile<HM, NT, EDGE>(acc[0], C, M, N, row0 + wm * 64, col0 + wn * 64, alpha);
    store_c_tile<HM, NT, EDGE>(acc[1], C, M, N, row0 + 128 + wm * 64, col0 + wn * 64, alpha);
}

}  // namespace hk
