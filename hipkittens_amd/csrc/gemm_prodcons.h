// Producer / consumer GEMM body (wave-specialised), shared by the FP8, BF16 and MXFP4 GEMMs (a K-step is
// 128 bytes per operand row in all three; only the MFMA differs).
//
// After the reference's wave-specialised micro kernel
// (kernels/gemm/bf16fp32/mi350x/micros/producer_consumer/32x16/micro_04_2stage_12c4p.cpp: 66-72 the split
// into a producer and three consumer groups of four waves, 88-101 the producers' preload, 107-137 the
// loop in which producers only load and consumers only multiply, one barrier per K-step, two LDS
// stages; tile 192 x 256 = 3 x 4 blocks of 64 x 64, one block per consumer wave): sixteen waves, four per
// SIMD (128 registers each),
//   waves 12..15  producers: all global->LDS loads of the next K-step's tiles (14 of the 56 1-KiB pieces each,
//                 plus the MXFP4 scale rows), then wait for them; nothing else;
//   waves 0..11   consumers: wave c owns the 64 x 64 block (c / 4, c % 4) of the 192 x 256 tile: it reads its
//                 four B fragments and, one at a time, its four A fragments from the current stage and issues
//                 the 16 MFMA tiles; it never issues or waits for a vector-memory load in the loop.
// Everybody meets at one barrier per K-step: the producers' tile has landed, the consumers have read theirs.
// What the hardware gives such a kernel here: the register file is divided evenly among a workgroup's waves,
// so the four producer waves hold a quarter of it for a handful of addresses, and a consumer's 64 x 64 block
// reads twice the LDS bytes per flop of the 4-wave kernels' 128 x 128 blocks. Measured next to the other
// two schedules (bench.py, leg `schedules`); the 4-wave kernels stay the default.
// Tile format, swizzle, B-row permutation, K tail and epilogue are those of the other tile kernels
// (gemm_tile.h); every output element sums its K-steps in the same order: identical bits.
#pragma once
#include "gemm_small_tile.h"

namespace hk {

constexpr int kPcBM = 192;                                  // tile rows (three consumer groups of 64)
constexpr int kPcATile = kPcBM * BK;                        // 24 KiB
constexpr int kPcStage = kPcATile + kTileBytes;             // A tile + B tile (56 KiB)
constexpr int kPcScaleSlot = (kPcBM + BN) * 16;             // MXFP4: 16 scale bytes (two K-steps) per row of A, then of B
constexpr int kPcLdsBytes = 2 * kPcStage;                   // 112 KiB
constexpr int kPcLdsBytesScaled = kPcLdsBytes + 2 * kPcScaleSlot;   // + two scale slots (14 KiB)
constexpr int kPcThreads = 16 * 64;

// MMA: as in gemm_small_tile_body (MMA::kScaled: MXFP4 with e8m0 scales in rows of sa_pitch / sb_pitch bytes,
// whole groups of 8 bytes). K: the operands' row length in BYTES (a multiple of 16).
template <typename MMA, bool EDGE>
__device__ __forceinline__ void gemm_prodcons_body(
    uint8_t* smem, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n,
    SmallTileScales sc = SmallTileScales{nullptr, nullptr, 0, 0}) {
    constexpr int NC = 12, NP = 4, MT = 4, NT = 4;
    constexpr int kAPieces = kPcATile / 1024, kBPieces = kTileBytes / 1024;   // 24 + 32 pieces of 8 rows
    static_assert(kAPieces % NP == 0 && kBPieces % NP == 0, "pieces per producer");
    constexpr bool kScaled = MMA::kScaled;
    const int lane = lane_id(), w = wave_id();
    const bool producer = w >= NC;

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        grouped_raster(id, tiles_m, tiles_n, 8, pm, pn);
    }
    const int row0 = pm * kPcBM, col0 = pn * BN;
    const int a_rows = min(M - row0, kPcBM), b_rows = min(N - col0, BN);
    const int nk = (K + BK - 1) / BK;
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;

    if (producer) {
        const int pw = w - NC;
        const v4i srd_a = make_srd(A + (size_t)row0 * K, (uint32_t)a_rows * (uint32_t)K);
        const v4i srd_b = make_srd(B + (size_t)col0 * K, (uint32_t)b_rows * (uint32_t)K);
        // piece i of this wave = tile rows 8 (NP i + pw) .. +8; lane l lands in row + l / 8, physical chunk l % 8
        uint32_t voff_a[kAPieces / NP], voff_b[kBPieces / NP];
#pragma unroll
        for (int i = 0; i < kAPieces / NP; ++i) {
            const int R = 8 * (i * NP + pw) + (lane >> 3);
            voff_a[i] = (uint32_t)(EDGE ? min(R, a_rows - 1) : R) * (uint32_t)K + swz_chunk(R, lane & 7) * 16u;
        }
#pragma unroll
        for (int i = 0; i < kBPieces / NP; ++i) {
            const int R = 8 * (i * NP + pw) + (lane >> 3);
            const int rb = b_row_to_col(R);
            voff_b[i] = (uint32_t)(EDGE ? min(rb, b_rows - 1) : rb) * (uint32_t)K + swz_chunk(R, lane & 7) * 16u;
        }
        const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)pw * 1024u);
        // last K-step of a K that is not a multiple of 128: lanes whose 16-byte chunk lies past the end of the
        // row go out of the buffer's range (bit 31) and write zeros. The chunk a lane fetches is the same for all
        // of its loads: swz(row, lane % 8) with row bits [1..3] = 4 pw + lane / 16 (mod 8)
        const uint32_t tail_or =
            (int)(swz_chunk(8 * pw + (lane >> 3), lane & 7) * 16u) >= K - (nk - 1) * BK ? 0x80000000u : 0u;
        // MXFP4 scale rows: seven groups of 64 rows (three of A, four of B), lane l row 64 j + l, 16 bytes = the
        // pair of K-steps kt / 2; producer pw fetches groups pw and pw + 4
        v4i srd_s[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
        uint32_t voff_s[2] = {0, 0}, lds_s[2] = {0, 0};
        if (kScaled) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int j = pw + 4 * q;          // group 0..6 (7: none)
                if (j >= 7) continue;
                const int op = j >= 3, srow0 = 64 * (op ? j - 3 : j);
                const int R = srow0 + lane;
                int rr = op ? b_row_to_col(R) : R;
                if (EDGE) rr = min(rr, (op ? b_rows : a_rows) - 1);
                const int pitch = op ? sc.sb_pitch : sc.sa_pitch;
                srd_s[q] = op ? make_srd(sc.SB + (size_t)col0 * pitch, (uint32_t)b_rows * (uint32_t)pitch)
                              : make_srd(sc.SA + (size_t)row0 * pitch, (uint32_t)a_rows * (uint32_t)pitch);
                voff_s[q] = (uint32_t)rr * (uint32_t)pitch;
                lds_s[q] = lds0 + kPcLdsBytes + (uint32_t)(op ? kPcBM * 16 : 0) + (uint32_t)srow0 * 16u;
            }
        }
        auto issue_tile = [&](int kt) {
            const uint32_t k0 = (uint32_t)kt * BK;
            const uint32_t dst = lds_wave + (uint32_t)(kt & 1) * kPcStage;
            const uint32_t vor = kt == nk - 1 ? tail_or : 0u;
#pragma unroll
            for (int i = 0; i < kAPieces / NP; ++i) dma16(srd_a, dst + i * NP * 1024, voff_a[i] | vor, k0);
#pragma unroll
            for (int i = 0; i < kBPieces / NP; ++i) dma16(srd_b, dst + kPcATile + i * NP * 1024, voff_b[i] | vor, k0);
            if (kScaled && (kt & 1) == 0) {
#pragma unroll
                for (int q = 0; q < 2; ++q)
                    if (pw + 4 * q < 7)
                        dma16(srd_s[q], to_sgpr(lds_s[q] + (uint32_t)((kt >> 1) & 1) * kPcScaleSlot), voff_s[q],
                              (uint32_t)(kt >> 1) * 16u);
            }
        };
        issue_tile(0);
        wait_vmcnt<0>();
        block_barrier();
        for (int kt = 0; kt < nk; ++kt) {
            if (kt + 1 < nk) issue_tile(kt + 1);
            wait_vmcnt<0>();
            block_barrier();   // the next tile has landed; the consumers have read this one
        }
        return;
    }

    // ---- consumers ------------------------------------------------------------------------------------
    const int cm = w >> 2, cn = w & 3;
    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    const uint32_t a_lo0 = lds0 + cm * (64 * BK) + rd_lo, a_hi0 = lds0 + cm * (64 * BK) + rd_hi;
    const uint32_t b_lo0 = lds0 + kPcATile + cn * (64 * BK) + rd_lo;
    const uint32_t b_hi0 = lds0 + kPcATile + cn * (64 * BK) + rd_hi;

    v4f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    block_barrier();   // the producers' first tile
    for (int kt = 0; kt < nk; ++kt) {
        const uint32_t so = (uint32_t)(kt & 1) * kPcStage;
        v8i bf[NT];
        v2i bs[NT];
        const uint32_t sh = 8u * g;
        // the lane's scale bytes: row 16 f + r of the wave's block, byte g of each K half's dword
        const uint32_t sbase = lds0 + kPcLdsBytes + (uint32_t)((kt >> 1) & 1) * kPcScaleSlot + (uint32_t)(kt & 1) * 8u + r * 16u;
#pragma unroll
        for (int n = 0; n < NT; ++n) bf[n] = lds_frag(b_lo0 + so, b_hi0 + so, n * 16 * BK);
        if constexpr (kScaled) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                bs[n] = *(lds_v2i_t*)(uintptr_t)(sbase + kPcBM * 16 + (cn * 64 + 16 * n) * 16);
                bs[n].x = (int)((uint32_t)bs[n].x >> sh); bs[n].y = (int)((uint32_t)bs[n].y >> sh);
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const v8i af = lds_frag(a_lo0 + so, a_hi0 + so, m * 16 * BK);
            if constexpr (kScaled) {
                v2i as = *(lds_v2i_t*)(uintptr_t)(sbase + (cm * 64 + 16 * m) * 16);
                as.x = (int)((uint32_t)as.x >> sh); as.y = (int)((uint32_t)as.y >> sh);
#pragma unroll
                for (int n = 0; n < NT; ++n) MMA::mma(acc[m][n], bf[n], af, bs[n], as);
            } else {
#pragma unroll
                for (int n = 0; n < NT; ++n) MMA::mma(acc[m][n], bf[n], af);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // (every read of this stage has returned)
        block_barrier();
    }
    store_c_tile<MT, NT, EDGE>(acc, C, M, N, row0 + cm * 64, col0 + cn * 64, alpha);
}

}  // namespace hk
