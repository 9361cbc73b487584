// Small-tile GEMM kernel body shared by the FP8 and BF16 GEMMs (a K-step is 128 bytes per operand
// row in both; only the MFMA differs).
#pragma once
#include "gemm_tile.h"
#include "hk_host.h"
#include "../../include/hk355.h"

namespace hk {

// 128x128-tile kernel body for problems with too few 256x256 tiles to occupy the chip (a 1024^3
// GEMM has 16 of them for 256 CUs): 4 waves, each a 64x64 patch (16 MFMA tiles), three LDS
// stages of 2 x 16 KiB with two K-steps of loads in flight, plain loop (such problems are
// bound by launch, prologue and epilogue latency, not by the K loop's schedule). Same tile
// format, B-row permutation and epilogue as the large-tile kernels.
constexpr int kSmallTile = 128;
constexpr int kSmallTileBytes = kSmallTile * BK;          // 16 KiB per operand
constexpr int kSmallStageBytes = 2 * kSmallTileBytes;
constexpr int kSmallStages = 3;
constexpr int kSmallLdsBytes = kSmallStages * kSmallStageBytes;  // 96 KiB
// the same kernel with 64x64 tiles and four 16 KiB stages (two workgroups per CU): for problems
// with so few 128x128 tiles that a quarter of the tile is needed to give every CU work
constexpr int kTinyTile = 64;
constexpr int kTinyStages = 4;
constexpr int kTinyLdsBytes = kTinyStages * 2 * kTinyTile * BK;  // 64 KiB

// SPLIT: blockIdx.y selects a range of `kps` K-steps; the tile's fp32 partial sums go to
// partial[blockIdx.y][M][N] (plain stores; splitk_reduce_kernel adds the ranges in order, so the
// result does not depend on timing). For problems with few tiles and a long K (decode-like
// shapes), where a single workgroup per tile walks K one K-step latency at a time.
// MMA: the operand type's MFMA on one 16-row x 128-byte fragment pair, `MMA::mma(acc, b, a)`. K is
// the operands' row length in BYTES (a multiple of 16); smem: the workgroup's dynamic LDS.
// MMA::kScaled (MXFP4): every operand row also has e8m0 block scales, 8 bytes per K-step, in rows of
// sa_pitch / sb_pitch bytes (multiples of 8); `MMA::mma(acc, b, a, sb, sa)` then takes, per fragment,
// the lane's scale bytes of the K-step's two halves in bits [7:0] of .x / .y.
// tail_pair / tail_shift: the pair of K-steps whose scale fetch starts tail_shift bytes early (rows that do not
// hold whole groups of 16 scale bytes; see mxfp4_gemm.hip), -1 / 0: none.
// row_bytes: scale bytes of a row that may be fetched (0: the whole pitch); the last row of an operand is in
// the descriptor's range up to there.
struct SmallTileScales {
    const uint8_t* SA; const uint8_t* SB; int sa_pitch, sb_pitch; int tail_pair = -1, tail_shift = 0, row_bytes = 0;
};
// bytes of the scale rows [row0, row0 + rows) that a descriptor covers
__device__ __forceinline__ uint32_t scale_rows_bytes(int rows, int pitch, int row_bytes) {
    return (uint32_t)(rows - 1) * (uint32_t)pitch + (uint32_t)(row_bytes ? row_bytes : pitch);
}
template <int TILE, int STAGES>
constexpr int small_tile_lds_bytes(bool scaled) { return STAGES * 2 * TILE * BK + (scaled ? 4 * 2 * TILE * 16 : 0); }

template <typename MMA, int TILE, int STAGES, bool EDGE, bool SPLIT>
__device__ __forceinline__ void gemm_small_tile_body(
    uint8_t* smem, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, int tiles_m, int tiles_n, int kps, float* __restrict__ partial,
    SmallTileScales sc = SmallTileScales{nullptr, nullptr, 0, 0}) {
    constexpr int NW = 4, TM = TILE / 2, TN = TILE / 2, MT = TM / 16, NT = TN / 16;
    constexpr int kTB = TILE * BK, kSB = 2 * kTB;    // bytes of one operand tile / of one stage
    constexpr int NDMA = kTB / (NW * 1024);          // loads per wave per operand per K-step
    constexpr bool kScaled = MMA::kScaled;
    constexpr int LPT = 2 * NDMA + (kScaled ? 1 : 0);  // loads per wave per K-step
    // scales: four slots, each the 16 bytes (two K-steps) of the TILE rows of A, then of B
    constexpr int kScaleSlot = 2 * TILE * 16, kScaleBase = STAGES * kSB;
    static_assert(STAGES >= 3 && STAGES <= 8 && (STAGES - 2) * LPT < 64, "vmcnt range");
    static_assert(!kScaled || STAGES <= 5, "four scale slots cover the K-step pairs of at most five stages");
    const int lane = lane_id(), w = wave_id();
    const int wm = w >> 1, wn = w & 1;

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        grouped_raster(id, tiles_m, tiles_n, 8, pm, pn);
    }
    const int row0 = pm * TILE, col0 = pn * TILE;
    const int a_rows = min(M - row0, TILE), b_rows = min(N - col0, TILE);
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
    // last K-step of a K that is not a multiple of 128: lanes whose 16-byte chunk lies past the
    // end of the row are moved out of the buffer's range (bit 31) and write zeros to LDS
    const uint32_t tail_or =
        (int)(swz_chunk(8 * w + (lane >> 3), lane & 7) * 16u) >= K - (nk - 1) * BK ? 0x80000000u : 0u;
    // this workgroup's K-steps: [kt0, kt0 + nkt)
    const int kt0 = SPLIT ? (int)blockIdx.y * kps : 0;
    const int nkt = SPLIT ? min(kps, nk - kt0) : nk;
    // Scale loads (kScaled): wave w fetches operand w & 1 (0 = A), lane l the 16 bytes of row
    // 64 (w >> 1) + l (TILE = 128; with TILE = 64 waves 2 and 3 repeat what 0 and 1 fetch), i.e. the
    // scales of the pair of K-steps kt / 2. Every wave issues one such load with every K-step (on odd
    // K-steps it repeats the pair's load into the same slot): the same number of loads per K-step in
    // every wave keeps the counted waits uniform.
    v4i srd_s = {0, 0, 0, 0};
    uint32_t voff_s = 0, lds_s = 0;
    if (kScaled) {
        const int op = w & 1, srow0 = TILE == 128 ? 64 * (w >> 1) : 0;
        const int R = srow0 + lane;
        int rr = op ? b_row_to_col(R) : R;
        if (EDGE) rr = min(rr, (op ? b_rows : a_rows) - 1);
        const int pitch = op ? sc.sb_pitch : sc.sa_pitch;
        srd_s = op ? make_srd(sc.SB + (size_t)col0 * pitch, scale_rows_bytes(b_rows, pitch, sc.row_bytes))
                   : make_srd(sc.SA + (size_t)row0 * pitch, scale_rows_bytes(a_rows, pitch, sc.row_bytes));
        voff_s = (uint32_t)rr * (uint32_t)pitch;
        lds_s = to_sgpr(lds0 + kScaleBase + (uint32_t)op * (TILE * 16) + (uint32_t)srow0 * 16u);
    }
    auto issue_tile = [&](int stage, int kt_local) {
        const int kt = kt0 + kt_local;
        const uint32_t k0 = (uint32_t)kt * BK;
        const uint32_t dst = lds_wave + (uint32_t)stage * kSB;
        const uint32_t vor = kt == nk - 1 ? tail_or : 0u;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma16(srd_a, dst + i * NW * 1024, voff_a[i] | vor, k0);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma16(srd_b, dst + kTB + i * NW * 1024, voff_b[i] | vor, k0);
        if (kScaled)
            dma16(srd_s, lds_s + (uint32_t)((kt >> 1) & 3) * kScaleSlot, voff_s,
                  (uint32_t)(kt >> 1) * 16u - ((kt >> 1) == sc.tail_pair ? (uint32_t)sc.tail_shift : 0u));
    };
    // wait until at most `tiles` of the most recently issued K-steps' loads are still in flight
    auto wait_tiles = [&](int tiles) {
        switch (tiles) {
            case 0: wait_vmcnt<0>(); break;
            case 1: wait_vmcnt<LPT>(); break;
            case 2: wait_vmcnt<(STAGES > 3 ? 2 : 1) * LPT>(); break;
            case 3: wait_vmcnt<(STAGES > 4 ? 3 : 1) * LPT>(); break;
            case 4: wait_vmcnt<(STAGES > 5 ? 4 : 1) * LPT>(); break;
            case 5: wait_vmcnt<(STAGES > 6 ? 5 : 1) * LPT>(); break;
            default: wait_vmcnt<(STAGES > 7 ? 6 : 1) * LPT>(); break;
        }
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    const uint32_t a_lo0 = lds0 + wm * (TM * BK) + rd_lo, a_hi0 = lds0 + wm * (TM * BK) + rd_hi;
    const uint32_t b_lo0 = lds0 + kTB + wn * (TN * BK) + rd_lo;
    const uint32_t b_hi0 = lds0 + kTB + wn * (TN * BK) + rd_hi;

    v4f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};

    // K-steps kt .. kt + STAGES - 2 are in flight or in LDS while step kt is multiplied
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if (p < nkt) issue_tile(p, p);
    int st = 0;
    for (int kt = 0; kt < nkt; ++kt) {
        // this wave's part of K-step kt has landed (the loads of the steps behind it may still fly)
        wait_tiles(min(nkt - 1 - kt, STAGES - 2));
        block_barrier();  // ... everyone's; and everyone is done with the stage of K-step kt - 1
        if (kt + STAGES - 1 < nkt) issue_tile(st == 0 ? STAGES - 1 : st - 1, kt + STAGES - 1);
        const uint32_t so = (uint32_t)st * kSB;
        v8i bf[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) bf[n] = lds_frag(b_lo0 + so, b_hi0 + so, n * 16 * BK);
        if constexpr (kScaled) {
            // the lane's scale bytes: row 16 f + r of the wave's patch, byte g of each half's dword
            const int ktg = kt0 + kt;
            const uint32_t sbase = lds0 + kScaleBase + (uint32_t)((ktg >> 1) & 3) * kScaleSlot + (uint32_t)(ktg & 1) * 8u + r * 16u +
                                   ((ktg >> 1) == sc.tail_pair ? (uint32_t)sc.tail_shift : 0u);
            const uint32_t sh = 8u * g;
            v2i bs[NT];
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                bs[n] = *(lds_v2i_t*)(uintptr_t)(sbase + TILE * 16 + (wn * TN + 16 * n) * 16);
                bs[n].x = (int)((uint32_t)bs[n].x >> sh); bs[n].y = (int)((uint32_t)bs[n].y >> sh);
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const v8i af = lds_frag(a_lo0 + so, a_hi0 + so, m * 16 * BK);
                v2i as = *(lds_v2i_t*)(uintptr_t)(sbase + (wm * TM + 16 * m) * 16);
                as.x = (int)((uint32_t)as.x >> sh); as.y = (int)((uint32_t)as.y >> sh);
#pragma unroll
                for (int n = 0; n < NT; ++n) MMA::mma(acc[m][n], bf[n], af, bs[n], as);
            }
        } else {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const v8i af = lds_frag(a_lo0 + so, a_hi0 + so, m * 16 * BK);
#pragma unroll
                for (int n = 0; n < NT; ++n) MMA::mma(acc[m][n], bf[n], af);
            }
        }
        st = st == STAGES - 1 ? 0 : st + 1;
    }
    if (!SPLIT) {
        store_c_tile<MT, NT, EDGE>(acc, C, M, N, row0 + wm * TM, col0 + wn * TN, alpha);
    } else {
        // fp32 partial sums: lane (r, g) holds, for row 16 m + r, columns 32 p + 8 g .. +8
        float* out = partial + (size_t)blockIdx.y * M * N;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = row0 + wm * TM + 16 * m + (int)r;
            if (row >= M) continue;
#pragma unroll
            for (int q = 0; q < NT / 2; ++q) {
                const int col = col0 + wn * TN + 32 * q + 8 * (int)g;
                float* dst = out + (size_t)row * N + col;
                if (col + 8 <= N && (N & 3) == 0) {
                    *(v4f*)dst = acc[m][2 * q];
                    *(v4f*)(dst + 4) = acc[m][2 * q + 1];
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (col + j < N) dst[j] = j < 4 ? acc[m][2 * q][j] : acc[m][2 * q + 1][j - 4];
                }
            }
        }
    }
}


// C = bf16(alpha * sum_s partial[s]) in split order; one thread per 4 columns.
static __global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits,
                                                            long long mn, float alpha,
                                                            uint16_t* __restrict__ C) {
    const long long i4 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= mn) return;
    if (i4 + 4 <= mn && (mn & 3) == 0) {
        v4f sum = *(const v4f*)(partial + i4);
        for (int s2 = 1; s2 < splits; ++s2) sum += *(const v4f*)(partial + (size_t)s2 * mn + i4);
        sum *= alpha;
        v2i o;
        o.x = pack_bf16(sum.x, sum.y); o.y = pack_bf16(sum.z, sum.w);
        *(v2i*)(C + i4) = o;
    } else {
        for (long long i = i4; i < mn && i < i4 + 4; ++i) {
            float sum = partial[i];
            for (int s2 = 1; s2 < splits; ++s2) sum += partial[(size_t)s2 * mn + i];
            C[i] = (uint16_t)(pack_bf16(sum * alpha, 0.f) & 0xffffu);
        }
    }
}

// Which tile a GEMM gets when the caller does not pin a kernel: 256 (the large-tile kernels), 128 or
// 64. Two layers:
//  1. a rule: the tile with the smallest estimated time. A tile kernel's workgroups run in rounds over the
//     device's CUs (one workgroup per CU for the 256- and 128-tiles, two for the 64-tile), every round costs
//     the same whether it is full or not, and a workgroup's time is a fixed part (prologue, epilogue, launch)
//     plus a part per K-step:  time = ceil(tiles / (CUs x workgroups per CU)) x (fixed + per_step x K-steps).
//     The two constants per tile and format were fitted to the sweep below on an MI355X (microseconds; they
//     enter only through their ratios, the CU count through the rounds). This captures what a threshold on the
//     tile count cannot: 72 tiles of 256 are one round where their 288 tiles of 128 are two (the large tile
//     wins by 4-12 % from a K of about 4096 elements on), 64 tiles of 256 are one round of four times the work
//     of the single round of 256 small tiles (the small tile wins by 60 %). Measured against the best of the
//     three kernels on 360 shapes per format, every launch on another copy of B (a model's weights come from HBM, not
//     from the memory-side cache), the rule alone is more than 5 % behind on 9 / 22 / 20 shapes (FP8 / BF16 /
//     MXFP4), mostly by 5 to 10 % where a long B is read by several rows of small tiles;
//  2. a generated table of the shapes on which a sweep found the rule's choice more than a few percent behind
//     another tile (tile_table.inc, written by `python -m hipkittens_amd.tile_sweep FORMAT --emit`; the
//     counterpart of the reference's per-shape analysis/baselines/gemm/utils/tuned.yaml). An entry is keyed by
//     the format, the numbers of 64-row / 64-column blocks of M and N and the K-step count, and applies on
//     devices with the CU count the sweep ran on.
struct TileRule {
    float fixed[3], per_step[3];   // 256-, 128-, 64-tile
};
enum TileFormat { kFmtFp8 = 0, kFmtBf16 = 1, kFmtMxfp4 = 2 };
struct TileTableEntry { unsigned char fmt; unsigned short m64, n64, nk, tile; };
#include "tile_table.inc"   // kTileTableCus, kTileTable[]

int moe_num_compute_units();  // number of CUs of the current device, cached (moe_mxfp4.hip)

static inline int pick_tile_rule(int M, int N, int nk, TileRule r, int cus) {
    const int tile[3] = {BM, kSmallTile, kTinyTile};
    const int per_cu[3] = {1, 1, 2};
    int best = 0;
    double best_time = 0.0;
    for (int i = 0; i < 3; ++i) {
        const long long tiles = (((long long)M + tile[i] - 1) / tile[i]) * (((long long)N + tile[i] - 1) / tile[i]);
        const long long capacity = (long long)cus * per_cu[i];
        const double time = (double)((tiles + capacity - 1) / capacity) * ((double)r.fixed[i] + (double)r.per_step[i] * nk);
        if (i == 0 || time < best_time) { best = i; best_time = time; }   // ties go to the larger tile
    }
    return tile[best];
}
static inline int pick_tile(int fmt, int M, int N, int nk, TileRule r, bool consult_table = true) {
    const int cus = moe_num_compute_units();   // 256 when no device can be queried
    if (consult_table && cus == kTileTableCus) {
        const long long m64 = ((long long)M + 63) / 64, n64 = ((long long)N + 63) / 64;
        for (const TileTableEntry& e : kTileTable)
            if (e.fmt == fmt && e.m64 == m64 && e.n64 == n64 && e.nk == nk) return e.tile;
    }
    // MXFP4, one row of 64x64 tiles and a wide output (128-column tiles for 7 of 8 CUs or more: N >= 28672 on 256
    // CUs): every 64-row tile fetches its own scale pieces, and with B streaming from HBM the 128x128 tile measured
    // 15 to 25 % faster at every K (M = 64, N = 32768, K = 16384: 85 -> 69 us), where the cost rule below, which
    // knows rounds and not bytes, takes the small tile
    if (fmt == kFmtMxfp4 && M <= kTinyTile && ((long long)N + kSmallTile - 1) / kSmallTile * 8 >= 7ll * cus) return kSmallTile;
    return pick_tile_rule(M, N, nk, r, cus);
}
// the formats' constants (K-steps: 128 bytes of an operand row)
constexpr TileRule kTileRuleFp8{{7.43f, 3.28f, 2.02f}, {1.078f, 0.585f, 0.372f}};
constexpr TileRule kTileRuleBf16{{7.75f, 3.15f, 2.17f}, {1.051f, 0.562f, 0.336f}};
constexpr TileRule kTileRuleMxfp4{{7.71f, 3.13f, 1.94f}, {1.316f, 0.767f, 0.549f}};

// Number of K ranges the split-K path would use: as many as fill the CUs, each at least 4
// K-steps long, at most 16; 1 = the problem has enough tiles or too short a K.
// K: the operands' row length in bytes; min_nk: the shortest K (in K-steps) that is split.
static inline int splitk_ranges(int M, int N, int K, int min_nk = 48) {
    // 64x64 tiles, two workgroups per CU
    // (64-bit: the size queries pass whatever the caller asks about)
    const long long tiles = (((long long)M + kTinyTile - 1) / kTinyTile) * (((long long)N + kTinyTile - 1) / kTinyTile);
    const long long nk = ((long long)K + BK - 1) / BK;
    const int cus = moe_num_compute_units();   // 256 when no device can be queried
    // shorter K: the 64x64-tile kernel without a second launch is as fast or faster; more than one tile for every
    // second CU: with B coming from HBM (every launch on another weight matrix) the split measured 5 to 25 % slower
    // than the plain kernel up to 128 K-steps, and within 8 % of it at 256
    if (tiles * 2 > cus || nk < min_nk) return 1;
    long long s = 2 * cus / tiles;
    if (s > nk / 4) s = nk / 4;
    if (s > 16) s = 16;
    return s < 2 ? 1 : (int)s;
}

// Launches `kern` (a small-tile kernel instantiated with SPLIT over 64x64 tiles) on `splits` K ranges
// and the reduction behind it. K in bytes.
template <typename Kern>
static inline int launch_small_tile_splitk(Kern kern, DeviceOnce& configured, const void* A, const void* B, void* C, int M,
                                           int N, int K, float alpha, int splits, float* partial,
                                           hipStream_t stream) {
    if (!set_lds_limit_once((const void*)kern, kTinyLdsBytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + kTinyTile - 1) / kTinyTile, tiles_n = (N + kTinyTile - 1) / kTinyTile;
    const int nk = (K + BK - 1) / BK;
    const int kps = (nk + splits - 1) / splits;
    const int used = (nk + kps - 1) / kps;   // ranges that hold at least one K-step
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n, used), dim3(256), kTinyLdsBytes, stream,
                       (const uint8_t*)A, (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha, tiles_m,
                       tiles_n, kps, partial);
    const long long mn = (long long)M * N;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((mn / 4 + 256) / 256)), dim3(256), 0, stream,
                       (const float*)partial, used, mn, alpha, (uint16_t*)C);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

}  // namespace hk
