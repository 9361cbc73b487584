// MXFP4 GEMM for gfx950: C[M,N] = bf16( sum_k A[m,k] * B[n,k] ), A and B in OCP MX format:
// e2m1 elements packed two per byte (even k in the low nibble) and one e8m0 scale per 32
// consecutive k (scales row-major [rows, K/32]); fp32 accumulation.
//
// No counterpart in the reference (it has no MXFP4 code); built on the same skeleton as the
// FP8 kernel (kernels/gemm/fp8fp32 in the reference) with the block scales applied inside
// the MFMA: v_mfma_scale_f32_16x16x128_f8f6f4 with cbsz = blgp = 4 (e2m1 operands) takes, per
// lane, one e8m0 byte for the lane's own 32-element K-block of each operand, which is exactly
// one MX block.
//
// Tile kernel: 256x256 tile of C, K-step 256 elements = 128 bytes per operand row, so the LDS
// tile layout, swizzle and read pattern are those of the FP8 kernel; the two 16-byte halves a
// lane reads per fragment row are MX blocks g and 4+g of the K-step and feed two MFMAs. The
// 8 scale bytes per row and K-step travel through LDS next to the tiles: one 16-byte direct load
// per row brings the scales of a pair of K-steps (every global->LDS load costs the CU's address
// unit the same time whatever its width, and that time is taken from the MFMAs, so the scales
// come in as few loads as possible: 2 per wave and pair of K-steps). They are read back with
// one ds_read_b64 per fragment and K-step; a per-lane shift moves byte g into the position the
// MFMA reads.
//
// Scale rows of any pitch and alignment (dense [rows, K / 32] rows for any K): a global->LDS load takes
// a source address of any byte alignment, so the only special case is the last pair of K-steps of a
// row that does not hold whole groups of 16 scale bytes. Its fetch would run past the end of the row
// and, for the last row of the array, past the array. That pair is fetched `tail_shift` (0..3) bytes
// early, so that a dword of the fetch ends exactly at the end of the row's scales: the dwords behind
// it are out of the descriptor's range for the last row (nothing is fetched, zeros land in LDS) and
// belong to K blocks past K otherwise; the readers add the same shift to their LDS address.
#include "gemm_tile.h"
#include "gemm_small_tile.h"
#include "gemm_pingpong.h"
#include "gemm_prodcons.h"
#include "gemm_skinny.h"
#include "../../include/hk355.h"

namespace hk {


constexpr int kScaleTileBytes = BM * 16;               // per row: 8 scale bytes for each K-step of a pair
constexpr int kScaleStageBytes = 2 * kScaleTileBytes;  // A + B
constexpr int kScaleBase = kLdsBytes;                  // scales sit behind the operand stages
constexpr int kLdsBytesFp4 = kLdsBytes + 2 * kScaleStageBytes;

// acc(16x16) += X(16x128 e2m1, scale sx) * Y(16x128 e2m1, scale sy)^T, accumulator tied in
// an AGPR; sx / sy carry the lane's e8m0 byte in bits [7:0].
__device__ __forceinline__ void mfma_fp4_acc(v4f& acc, const v4i& x, const v4i& y, int sx, int sy) {
    asm volatile(
        "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
        : "+a"(acc)
        : "v"(x), "v"(y), "v"(sx), "v"(sy));
}

template <bool EDGE>
__global__ __launch_bounds__(256) void mxfp4_gemm_4wave_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch,
    int sb_pitch, int tiles_m, int tiles_n, int band_n, int tail_pair, int tail_shift, int scale_row_bytes) {
    constexpr int NW = 4, TM = 128, TN = 128, MT = 8, NT = 8;
    constexpr int NDMA = kTileBytes / (NW * 1024);
    constexpr int PG = 4, AD = 3;
    static_assert(PG == 4 && AD == 3 && MT == 8, "slot plan below is written for these");
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];

    const int lane = lane_id();
    const int w = wave_id();
    const int wm = w >> 1, wn = w & 1;
    const int Kb = K >> 1;   // operand row pitch in bytes (scale rows: sa_pitch / sb_pitch bytes)

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        banded_raster(id, tiles_m, tiles_n, band_n < tiles_n ? 4 : 8, band_n, pm, pn);
    }
    const int row0 = pm * BM, col0 = pn * BN;
    const int a_rows = min(M - row0, BM), b_rows = min(N - col0, BN);
    const v4i srd_a = make_srd(A + (size_t)row0 * Kb, (uint32_t)a_rows * (uint32_t)Kb);
    const v4i srd_b = make_srd(B + (size_t)col0 * Kb, (uint32_t)b_rows * (uint32_t)Kb);
    const v4i srd_sa = make_srd(SA + (size_t)row0 * sa_pitch, scale_rows_bytes(a_rows, sa_pitch, scale_row_bytes));
    const v4i srd_sb = make_srd(SB + (size_t)col0 * sb_pitch, scale_rows_bytes(b_rows, sb_pitch, scale_row_bytes));

    // operand tiles: as in the FP8 kernel
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
    // scale tiles: this wave loads LDS rows 64w..64w+63 of each operand, lane l -> row 64w + l,
    // 16 bytes = the row's scales of K-steps 2p and 2p+1
    uint32_t voff_sa, voff_sb;
    {
        const int R = 64 * w + lane;
        int ra = R, rb = b_row_to_col(R);
        if (EDGE) {
            ra = min(ra, a_rows - 1);
            rb = min(rb, b_rows - 1);
        }
        voff_sa = (uint32_t)ra * (uint32_t)sa_pitch;
        voff_sb = (uint32_t)rb * (uint32_t)sb_pitch;
    }
    const uint32_t dma_row_stride = to_sgpr((uint32_t)(8 * NW) * (uint32_t)Kb);
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const uint32_t lds_scale_wave = to_sgpr(lds0 + kScaleBase + (uint32_t)w * 1024u);

    // `vor`: 0, or in the last K-step of a K that is not a multiple of 256 bit 31 for the lanes whose
    // 16 bytes lie past the end of the row: out of the buffer's range, so zeros land in LDS
    auto dma_one = [&](int op, int i, int stage, uint32_t k0, v4i srd, uint32_t vor) {
        const uint32_t dst = lds_wave + (uint32_t)stage * kStageBytes + op * kTileBytes + i * NW * 1024;
        if (EDGE)
            dma16(srd, dst, (op ? voff_b[i] : voff_a[i]) | vor, k0);
        else
            dma16(srd, dst, (op ? voff_b[0] : voff_a[0]) | vor, k0 + i * dma_row_stride);
    };
    // this wave's scale load of operand `op` for the pair of K-steps `pair` (stage pair % 2)
    auto dma_scale = [&](int op, uint32_t pair, v4i srd) {
        const uint32_t dst = lds_scale_wave + (pair & 1u) * kScaleStageBytes + op * kScaleTileBytes;
        dma16(srd, dst, op ? voff_sb : voff_sa, pair * 16u - ((int)pair == tail_pair ? (uint32_t)tail_shift : 0u));
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    uint32_t a_lo[2], a_hi[2], b_lo[2], b_hi[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
        a_lo[st] = lds0 + st * kStageBytes + wm * (TM * BK) + rd_lo;
        a_hi[st] = lds0 + st * kStageBytes + wm * (TM * BK) + rd_hi;
        b_lo[st] = lds0 + st * kStageBytes + kTileBytes + wn * (TN * BK) + rd_lo;
        b_hi[st] = lds0 + st * kStageBytes + kTileBytes + wn * (TN * BK) + rd_hi;
    }
    // scales of fragment f, K-step parity p, in the stage of the pair the base points to:
    // base + f*256 + p*8; sa_rd / sb_rd follow the pair of the running K-step
    uint32_t sa_rd = lds0 + kScaleBase + (wm * TM + r) * 16u;
    uint32_t sb_rd = lds0 + kScaleBase + kScaleTileBytes + (wn * TN + r) * 16u;
    static_assert(kScaleBase % (2 * kScaleStageBytes) == 0, "the pair's stage is toggled with xor");
    asm volatile("" : "+v"(sa_rd), "+v"(sb_rd));  // keep the large base in the register, offsets in immediates
    const uint32_t sh = 8u * g;  // byte g of each scale dword belongs to this lane
    auto rd_scale = [&](uint32_t base, int p, int f) -> v2i {
        return *(lds_v2i_t*)(uintptr_t)(base + f * 256 + p * 8);
    };
    auto shift_scale = [&](v2i& s) {
        s.x = (int)((uint32_t)s.x >> sh);
        s.y = (int)((uint32_t)s.y >> sh);
    };

    v4f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
    Frag4 bf[2][NT], af[4];
    v2i bs[2][NT], as[4];

    const int nk = (Kb + BK - 1) / BK;
    // the chunk a lane fetches is the same for all of its loads (see the FP8 kernel)
    const uint32_t tail_or =
        (int)(swz_chunk(8 * w + (lane >> 3), lane & 7) * 16u) >= Kb - (nk - 1) * BK ? 0x80000000u : 0u;

    // ---- prologue ----------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < NDMA; ++i) dma_one(0, i, 0, 0, srd_a, nk == 1 ? tail_or : 0u);
#pragma unroll
    for (int i = 0; i < NDMA; ++i) dma_one(1, i, 0, 0, srd_b, nk == 1 ? tail_or : 0u);
    dma_scale(0, 0, srd_sa);
    dma_scale(1, 0, srd_sb);
    wait_vmcnt<0>();
    block_barrier();
    if (nk > 1) {
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_one(0, i, 1, BK, srd_a, nk == 2 ? tail_or : 0u);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma_one(1, i, 1, BK, srd_b, nk == 2 ? tail_or : 0u);
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        bf[0][n] = lds_frag4(b_lo[0], b_hi[0], n * 16 * BK);
        bs[0][n] = rd_scale(sb_rd, 0, n);
    }
#pragma unroll
    for (int m = 0; m < AD; ++m) {
        af[m] = lds_frag4(a_lo[0], a_hi[0], m * 16 * BK);
        as[m] = rd_scale(sa_rd, 0, m);
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) shift_scale(bs[0][n]);
    shift_scale(as[0]);  // as[1], as[2] are shifted inside the first step (groups 0 and 1)

    // One K-step (slot plan of gemm_ring.h over two LDS stages). Scale handling: the raw
    // 8 bytes of a fragment are read together with the fragment; the shift that exposes
    // this lane's byte is placed well after the read (B: group 7; A fragment f: group f-1).
    // A scaled FP4 MFMA of this shape runs 16 cycles and keeps the wave's issue busy for about 12 of
    // them: one other instruction per MFMA is free, a second one already delays the next MFMA (register-only
    // loop, one wave per SIMD, cycles per MFMA with 0 / 1 / 2 / 3 independent v_add behind each: 16.8 / 17.1 /
    // 21.2 / 27.4; the unscaled FP8 form, 32 cycles, takes five before it slows down). Hence at most two
    // instructions per slot below, spread over both passes. (The same kernel on the 32x32x64 form of the
    // instruction, 64 MFMAs of 32 cycles per K-step with room for four instructions each and no per-lane
    // shifts, was built and measured: 8192^3 on all-zero operands 5840 against 5700 TFLOP/s, on random
    // operands 4550 against 4730: the accumulators' traffic per flop doubles, and with operands that toggle
    // the part is power limited.)
    auto step = [&]<int P>(int kt) {
        const uint32_t k2 = (uint32_t)(kt + 2) * BK;
        v4i sa = srd_a, sb = srd_b, ssa = srd_sa, ssb = srd_sb;
        if (kt + 2 >= nk) { sa.z = 0; sb.z = 0; ssa.z = 0; ssb.z = 0; }
        const uint32_t vor = kt + 2 == nk - 1 ? tail_or : 0u;
        // scales of the next K-step: same pair (P == 0) or the next pair, in the other stage
        // (entering the pair that was fetched tail_shift bytes early: see the head of the file)
        const uint32_t early = P && ((kt + 1) >> 1) == tail_pair ? (uint32_t)tail_shift : 0u;
        const uint32_t sa_nx = P ? (sa_rd ^ kScaleStageBytes) + early : sa_rd;
        const uint32_t sb_nx = P ? (sb_rd ^ kScaleStageBytes) + early : sb_rd;
        // operations behind the barrier, spread over the 48 MFMAs of both passes of groups 5..7: slot q
        // (0..47) = 16 (m - 5) + 8 pass + n. Global->LDS loads at q = 0, 3, .., 45 (the pair's scale loads at
        // 46, 47); LDS reads in the two slots between: unit u (fragment in the first, its scales in the
        // second) = B0..B4, A0, B5, B6, B7, A1, -, A2 (A fragment j's registers are free once group 4 + j is done)
        auto post_ops = [&](int q) __attribute__((always_inline)) {
            if (q % 3 == 0) {
                const int i = q / 3;
                dma_one(i / NDMA, i % NDMA, P, k2, i / NDMA ? sb : sa, vor);
            } else if (P == 0 && q >= 46) {
                dma_scale(q - 46, (uint32_t)(kt >> 1) + 1u, q - 46 ? ssb : ssa);
            }
            if (q % 3 != 0) {
                const int u = q / 3, part = q % 3 - 1;
                constexpr int kUnit[16] = {0, 1, 2, 3, 4, 8, 5, 6, 7, 9, -1, 10, -1, -1, -1, -1};   // 0..7: B, 8..10: A
                const int x = kUnit[u];
                if (x >= 0 && x < 8) {
                    if (part == 0) bf[P ^ 1][x] = lds_frag4(b_lo[P ^ 1], b_hi[P ^ 1], x * 16 * BK);
                    else bs[P ^ 1][x] = rd_scale(sb_nx, P ^ 1, x);
                } else if (x >= 8) {
                    if (part == 0) af[x - 8] = lds_frag4(a_lo[P ^ 1], a_hi[P ^ 1], (x - 8) * 16 * BK);
                    else as[x - 8] = rd_scale(sa_nx, P ^ 1, x - 8);
                }
            }
        };
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            // first the 8 MFMAs on the low K-half (MX block g), then the 8 on the high half
            // (block 4+g): the two MFMAs into one accumulator are 8 issue slots apart
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                mfma_fp4_acc(acc[m][n], bf[P][n].lo, af[m & 3].lo, bs[P][n].x, as[m & 3].x);
                if (m <= PG) {
                    if (n == 0) {
                        af[(m + AD) & 3] = lds_frag4(a_lo[P], a_hi[P], (m + AD) * 16 * BK);
                        as[(m + AD) & 3] = rd_scale(sa_rd, P, m + AD);
                    }
                } else {
                    post_ops((m - PG - 1) * 16 + n);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                mfma_fp4_acc(acc[m][n], bf[P][n].hi, af[m & 3].hi, bs[P][n].y, as[m & 3].y);
                if (m > PG) post_ops((m - PG - 1) * 16 + 8 + n);
                if (m == MT - 1) shift_scale(bs[P ^ 1][n]);
                // scale of A fragment m+1 (next step's fragment 0 when m == 7)
                if (n == 4) shift_scale(as[(m + 1) & 3]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                wait_vmcnt<0>();
                block_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (P) {
            sa_rd = sa_nx;
            sb_rd = sb_nx;
        }
    };

    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        step.template operator()<0>(kt);
        step.template operator()<1>(kt + 1);
    }
    if (kt < nk) step.template operator()<0>(kt);
    wait_vmcnt<0>();
    mfma_drain_agpr(acc);

    store_c_tile<MT, NT, EDGE>(acc, C, M, N, row0 + wm * TM, col0 + wn * TN, 1.0f);
}

// Portable kernel for any M, N and K % 32 == 0: operands and scales straight from global
// memory, K-step 128 elements (lane group g holds MX block g of the step).
__global__ __launch_bounds__(256) void mxfp4_gemm_portable_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch, int sb_pitch) {
    const int lane = lane_id(), w = wave_id();
    const int r = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.y * 64 + (w >> 1) * 32;
    const int col0 = blockIdx.x * 64 + (w & 1) * 32;
    const int Kb = K >> 1;
    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < K; k0 += 128) {
        v4i af[2], bf[2];
        int as[2], bs[2];
        const int kk = k0 + 32 * g;  // first element of this lane's block
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int ra = row0 + 16 * i + r, rb = col0 + 16 * i + r;
            af[i] = v4i{0, 0, 0, 0}; bf[i] = v4i{0, 0, 0, 0};
            as[i] = 127; bs[i] = 127;
            if (ra < M && kk < K) {
                af[i] = *(const v4i*)(A + (size_t)ra * Kb + (kk >> 1));
                as[i] = SA[(size_t)ra * sa_pitch + (kk >> 5)];
            }
            if (rb < N && kk < K) {
                bf[i] = *(const v4i*)(B + (size_t)rb * Kb + (kk >> 1));
                bs[i] = SB[(size_t)rb * sb_pitch + (kk >> 5)];
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma_fp4(bf[j], af[i], acc[i][j], bs[j], as[i]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = row0 + 16 * i + r;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float v[4] = {acc[i][j].x, acc[i][j].y, acc[i][j].z, acc[i][j].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = col0 + 16 * j + 4 * g + e;
                if (row < M && col < N)
                    C[(size_t)row * N + col] = (uint16_t)(pack_bf16(v[e], 0.f) & 0xffffu);
            }
        }
    }
}

// Small-tile kernels (gemm_small_tile.h) with the scaled FP4 MFMA, for problems with too few 256x256
// tiles to occupy the chip: the two 16-byte halves of a fragment row are MX blocks g and 4 + g of
// the 256-element K-step.
struct Mxfp4Mma {
    static constexpr bool kScaled = true;
    static __device__ __forceinline__ void mma(v4f& acc, const v8i& b, const v8i& a, const v2i& sb, const v2i& sa) {
        const v4i blo = {b[0], b[1], b[2], b[3]}, bhi = {b[4], b[5], b[6], b[7]};
        const v4i alo = {a[0], a[1], a[2], a[3]}, ahi = {a[4], a[5], a[6], a[7]};
        acc = mfma_fp4(blo, alo, acc, sb.x, sa.x);
        acc = mfma_fp4(bhi, ahi, acc, sb.y, sa.y);
    }
};
// K: the operands' row length in bytes (two elements per byte).
template <int TILE, int STAGES, bool EDGE, bool SPLIT = false>
__global__ __launch_bounds__(256) void mxfp4_gemm_small_tile_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch,
    int sb_pitch, int tiles_m, int tiles_n, int kps, float* __restrict__ partial, int tail_pair, int tail_shift,
    int scale_row_bytes) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_small_tile_body<Mxfp4Mma, TILE, STAGES, EDGE, SPLIT>(
        smem, A, B, C, M, N, K, 1.0f, tiles_m, tiles_n, kps, partial,
        SmallTileScales{SA, SB, sa_pitch, sb_pitch, tail_pair, tail_shift, scale_row_bytes});
}

// The skinny kernel (gemm_skinny.h) with the scaled FP4 MFMA, for at most 64 rows of A. K: the operands' row
// length in bytes; scale rows of any pitch and alignment, row_bytes scale bytes each.
template <int R, int NW, int D, int NF, bool NT>
__global__ __launch_bounds__(64 * NW) void mxfp4_gemm_skinny_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch, int sb_pitch,
    int row_bytes) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_skinny_body<Mxfp4Mma, R, NW, D, NF, NT>(smem, A, B, C, M, N, K, 1.0f, SkinnyScales{SA, SB, sa_pitch, sb_pitch, row_bytes});
}
template <int R, int NW, int D, int NF, bool NT>
static int launch_mxfp4_skinny_kernel(const void* A, const void* SA, const void* B, const void* SB, void* C, int M,
                                      int N, int K, int sa_pitch, int sb_pitch, hipStream_t stream) {
    auto kern = mxfp4_gemm_skinny_kernel<R, NW, D, NF, NT>;
    constexpr int lds_bytes = skinny_lds_bytes(R, NW, D, true, NF);
    static_assert(lds_bytes <= 160 * 1024, "LDS of one CU");
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((N + 16 * NF - 1) / (16 * NF)), dim3(64 * NW), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB, (uint16_t*)C, M, N, K / 2, sa_pitch,
                       sb_pitch, K / 32);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}
// rows of B per workgroup and the non-temporal hint as for the other formats (HK_SKINNY_DISPATCH)
template <int R, int NW, int D>
static int launch_mxfp4_skinny_pick(const void* A, const void* SA, const void* B, const void* SB, void* C, int M, int N,
                                    int K, int sa_pitch, int sb_pitch, hipStream_t stream) {
    const bool nf1 = 2ll * ((N + 31) / 32) <= moe_num_compute_units();
    const bool nt = (long long)N * (K / 2) >= kSkinnyNtBytes;
    if (nf1) return nt ? launch_mxfp4_skinny_kernel<R, NW, D, 1, true>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream)
                       : launch_mxfp4_skinny_kernel<R, NW, D, 1, false>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream);
    return nt ? launch_mxfp4_skinny_kernel<R, NW, D, 2, true>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream)
              : launch_mxfp4_skinny_kernel<R, NW, D, 2, false>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream);
}
static int launch_mxfp4_skinny(const void* A, const void* SA, const void* B, const void* SB, void* C, int M, int N,
                               int K, int sa_pitch, int sb_pitch, hipStream_t stream) {
    if (M <= 16) return launch_mxfp4_skinny_pick<1, 4, 4>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream);
    if (M <= 32) return launch_mxfp4_skinny_pick<2, 4, 3>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream);
    return launch_mxfp4_skinny_pick<4, 2, 4>(A, SA, B, SB, C, M, N, K, sa_pitch, sb_pitch, stream);
}

// What the tile kernels need to know about the scale rows (see the head of the file).
// ok: the tile kernels can take these rows; tail_pair / tail_shift: the pair of K-steps fetched early and by how
// many bytes (-1 / 0: none); row_bytes: what the scale descriptors cover of an operand's last row (0: its pitch).
struct Mxfp4ScaleRows { bool ok; int tail_pair, tail_shift, row_bytes; };
static Mxfp4ScaleRows mxfp4_scale_rows(int K, int sa_pitch, int sb_pitch) {
    const int nb = K / 32;                       // scale bytes of a row
    const int groups = (nb + 7) / 8 * 8;
    if (sa_pitch < nb || sb_pitch < nb) return {false, -1, 0, 0};
    // rows padded to whole groups of 8 bytes: a pair's fetch stays inside the row or ends on a dword of it
    if ((sa_pitch % 8) == 0 && (sb_pitch % 8) == 0 && sa_pitch >= groups && sb_pitch >= groups) return {true, -1, 0, 0};
    // any other pitch: nothing past a row's nb bytes is relied on, and the last row ends there. Rows of fewer than
    // 16 bytes (K < 512) stay with the portable kernel: the early fetch would start in front of the first row, and
    // the fetch of a row before the last could reach across the last one to the end of the array.
    if (nb < 16) return {false, -1, 0, 0};
    const int shift = (4 - nb % 4) % 4;
    if ((nb % 16) == 0 || shift == 0) return {true, -1, 0, nb};
    return {true, (nb - 1) / 16, shift, nb};
}

template <int TILE, int STAGES, bool EDGE>
static int launch_mxfp4_small_tile(const void* A, const void* SA, const void* B, const void* SB, void* C,
                                   int M, int N, int K, int sa_pitch, int sb_pitch, Mxfp4ScaleRows sr,
                                   hipStream_t stream) {
    auto kern = mxfp4_gemm_small_tile_kernel<TILE, STAGES, EDGE>;
    constexpr int lds_bytes = small_tile_lds_bytes<TILE, STAGES>(true);
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + TILE - 1) / TILE, tiles_n = (N + TILE - 1) / TILE;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB, (uint16_t*)C, M, N, K / 2,
                       sa_pitch, sb_pitch, tiles_m, tiles_n, 0, (float*)nullptr, sr.tail_pair, sr.tail_shift,
                       sr.row_bytes);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// Split-K over 64x64 tiles for problems with few tiles and a long K (decode shapes): `splits` K ranges of
// an even number of K-steps each (a range then starts on a pair of K-steps, the unit of a scale load),
// fp32 partial sums, and the fixed-order reduction behind them. K in elements.
constexpr int kMxfp4SplitMinSteps = 16;
// Number of K ranges for the MXFP4 GEMM (1: not split). On top of the common rule: at least four ranges
// (fewer only occur when the plain kernel already keeps more than half of the CUs busy: measured slower),
// and the time saved, 0.4 us per K-step taken off a workgroup's K loop, must exceed the second launch
// (2.5 us) and writing and reading the partial sums at 4 TB/s (M = 128, N = K = 4096: 9.0 us plain,
// 10.9 us split four ways, so not split; M = 16: 8.6 -> 6.6 us).
static int mxfp4_splitk_ranges(int M, int N, int K) {
    const int s = splitk_ranges(M, N, K / 2, kMxfp4SplitMinSteps);
    if (s < 4) return 1;
    const int nk = (K / 2 + BK - 1) / BK;
    const double saved_us = 0.4 * nk * (1.0 - 1.0 / s);
    const double cost_us = 2.5 + 8.0 * s * (double)M * (double)N / 4e6;
    return saved_us > cost_us ? s : 1;
}
template <bool EDGE>
static int launch_mxfp4_splitk(const void* A, const void* SA, const void* B, const void* SB, void* C, int M, int N,
                               int K, int sa_pitch, int sb_pitch, Mxfp4ScaleRows sr, int splits, float* partial,
                               hipStream_t stream) {
    auto kern = mxfp4_gemm_small_tile_kernel<kTinyTile, kTinyStages, EDGE, true>;
    constexpr int lds_bytes = small_tile_lds_bytes<kTinyTile, kTinyStages>(true);
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + kTinyTile - 1) / kTinyTile, tiles_n = (N + kTinyTile - 1) / kTinyTile;
    const int nk = (K / 2 + BK - 1) / BK;
    const int kps = ((nk + splits - 1) / splits + 1) & ~1;
    const int used = (nk + kps - 1) / kps;   // ranges that hold at least one K-step
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n, used), dim3(256), lds_bytes, stream, (const uint8_t*)A,
                       (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB, (uint16_t*)C, M, N, K / 2,
                       sa_pitch, sb_pitch, tiles_m, tiles_n, kps, partial, sr.tail_pair, sr.tail_shift, sr.row_bytes);
    const long long mn = (long long)M * N;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((mn / 4 + 256) / 256)), dim3(256), 0, stream,
                       (const float*)partial, used, mn, 1.0f, (uint16_t*)C);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// 8-wave ping-pong kernel (gemm_pingpong.h) with the scaled FP4 MFMA. K: the operands' row length in bytes.
template <bool EDGE>
__global__ __launch_bounds__(512) void mxfp4_gemm_pingpong_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch,
    int sb_pitch, int tiles_m, int tiles_n, int band_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_pingpong_body<Mxfp4Mma, EDGE>(smem, A, B, C, M, N, K, 1.0f, tiles_m, tiles_n, band_n,
                                       SmallTileScales{SA, SB, sa_pitch, sb_pitch});
}

// Producer / consumer kernel (gemm_prodcons.h) with the scaled FP4 MFMA. K: the operands' row length in bytes.
template <bool EDGE>
__global__ __launch_bounds__(kPcThreads) void mxfp4_gemm_prodcons_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ SA, const uint8_t* __restrict__ B,
    const uint8_t* __restrict__ SB, uint16_t* __restrict__ C, int M, int N, int K, int sa_pitch,
    int sb_pitch, int tiles_m, int tiles_n) {
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    gemm_prodcons_body<Mxfp4Mma, EDGE>(smem, A, B, C, M, N, K, 1.0f, tiles_m, tiles_n,
                                       SmallTileScales{SA, SB, sa_pitch, sb_pitch});
}

template <bool EDGE>
static int launch_mxfp4_prodcons(const void* A, const void* SA, const void* B, const void* SB, void* C,
                                 int M, int N, int K, int sa_pitch, int sb_pitch, hipStream_t stream) {
    auto kern = mxfp4_gemm_prodcons_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPcLdsBytesScaled, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + kPcBM - 1) / kPcBM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kPcThreads), kPcLdsBytesScaled, stream,
                       (const uint8_t*)A, (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB,
                       (uint16_t*)C, M, N, K / 2, sa_pitch, sb_pitch, tiles_m, tiles_n);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <bool EDGE>
static int launch_mxfp4_pingpong(const void* A, const void* SA, const void* B, const void* SB, void* C,
                                 int M, int N, int K, int sa_pitch, int sb_pitch, hipStream_t stream) {
    auto kern = mxfp4_gemm_pingpong_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kPpLdsBytesScaled, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(512), kPpLdsBytesScaled, stream,
                       (const uint8_t*)A, (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB,
                       (uint16_t*)C, M, N, K / 2, sa_pitch, sb_pitch, tiles_m, tiles_n,
                       raster_band(((long long)M + N) * (K / 2), tiles_n));
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

template <bool EDGE>
static int launch_mxfp4_4wave(const void* A, const void* SA, const void* B, const void* SB, void* C,
                              int M, int N, int K, int sa_pitch, int sb_pitch, Mxfp4ScaleRows sr, hipStream_t stream) {
    auto kern = mxfp4_gemm_4wave_kernel<EDGE>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kLdsBytesFp4, configured)) return HK_ERR_LAUNCH;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), kLdsBytesFp4, stream,
                       (const uint8_t*)A, (const uint8_t*)SA, (const uint8_t*)B, (const uint8_t*)SB,
                       (uint16_t*)C, M, N, K, sa_pitch, sb_pitch, tiles_m, tiles_n,
                       raster_band(((long long)M + N) * (K / 2), tiles_n), sr.tail_pair, sr.tail_shift, sr.row_bytes);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

}  // namespace hk

// variant: -1 = choose, 0 = portable kernel, 1 = 256x256 tile kernel (4 waves), 2 / 3 = 128x128 / 64x64 tiles,
// 4 = 256x256 tile kernel with the 8-wave ping-pong schedule, 5 = 192x256 tile producer / consumer kernel,
// 6 = the skinny kernel (at most 64 rows of A).
// Scale rows are sa_pitch / sb_pitch bytes apart (>= K / 32).
static int mxfp4_gemm_impl(const void* A, const void* A_scales, int sa_pitch, const void* B, const void* B_scales,
                           int sb_pitch, void* C, int M, int N, int K, int variant, void* stream) {
    using namespace hk;
    if (!A || !A_scales || !B || !B_scales || !C) return HK_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 32) != 0 || sa_pitch < K / 32 || sb_pitch < K / 32 ||
        gemm_dims_too_large(M, N, K))
        return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (variant < -1 || variant > 6) return HK_ERR_UNSUPPORTED;
    if (variant == 6 && M > kSkinnyMaxMScaled) return HK_ERR_UNSUPPORTED;
    // what the tile kernels need of the scale rows (any pitch and alignment; see mxfp4_scale_rows)
    const Mxfp4ScaleRows sr = mxfp4_scale_rows(K, sa_pitch, sb_pitch);
    const bool size_ok = (long long)(K / 2) * BM < (1ll << 31) && (long long)BM * max(sa_pitch, sb_pitch) < (1ll << 31);
    if (variant < 0) {
        // the choice of tile of hk_fp8_gemm (pick_tile); a K-step is 256 elements here
        const int tile = pick_tile(kFmtMxfp4, M, N, (K / 2 + BK - 1) / BK, kTileRuleMxfp4);
        variant = !(sr.ok && size_ok) ? 0 : tile == kTinyTile ? 3 : tile == kSmallTile ? 2 : 1;
        // few rows: one pass over B by the skinny kernel where that is faster (use_skinny); it takes any scale rows
        if (size_ok && use_skinny(M, N, (K / 2 + BK - 1) / BK, false, moe_num_compute_units(), kSkinnyMaxMScaled, 2)) variant = 6;
    }
    hipStream_t s = (hipStream_t)stream;
    if (variant == 0) {
        if ((M + 63) / 64 > 65535) return HK_ERR_BAD_SHAPE;
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        hipLaunchKernelGGL(mxfp4_gemm_portable_kernel, grid, dim3(256), 0, s, (const uint8_t*)A,
                           (const uint8_t*)A_scales, (const uint8_t*)B, (const uint8_t*)B_scales,
                           (uint16_t*)C, M, N, K, sa_pitch, sb_pitch);
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
    }
    if (variant == 6) {
        if (!size_ok) return HK_ERR_BAD_SHAPE;
        return launch_mxfp4_skinny(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, s);
    }
    if (!size_ok || !sr.ok) return HK_ERR_BAD_SHAPE;
    if (variant == 2) {
        const bool e = (M % kSmallTile) != 0 || (N % kSmallTile) != 0;
        return e ? launch_mxfp4_small_tile<kSmallTile, kSmallStages, true>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s)
                 : launch_mxfp4_small_tile<kSmallTile, kSmallStages, false>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s);
    }
    if (variant == 3) {
        const bool e = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
        return e ? launch_mxfp4_small_tile<kTinyTile, kTinyStages, true>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s)
                 : launch_mxfp4_small_tile<kTinyTile, kTinyStages, false>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s);
    }
    const bool edge = (M % BM) != 0 || (N % BN) != 0;
    if (variant == 4 || variant == 5) {
        // the ping-pong and producer / consumer kernels keep the padded-row form (rows of whole groups of 8 scale bytes)
        if (sr.row_bytes != 0) return HK_ERR_BAD_SHAPE;
        if (((uintptr_t)A_scales | (uintptr_t)B_scales) & 3u) return HK_ERR_BAD_ALIGNMENT;
        if (variant == 5) {
            const bool e = (M % kPcBM) != 0 || (N % BN) != 0;
            return e ? launch_mxfp4_prodcons<true>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, s)
                     : launch_mxfp4_prodcons<false>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, s);
        }
        return edge ? launch_mxfp4_pingpong<true>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, s)
                    : launch_mxfp4_pingpong<false>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, s);
    }
    return edge ? launch_mxfp4_4wave<true>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s)
                : launch_mxfp4_4wave<false>(A, A_scales, B, B_scales, C, M, N, K, sa_pitch, sb_pitch, sr, s);
}

extern "C" int hk_mxfp4_gemm_variant(const void* A, const void* A_scales, const void* B,
                                     const void* B_scales, void* C, int M, int N, int K, int variant,
                                     void* stream) {
    if (variant < 0) return HK_ERR_UNSUPPORTED;
    return mxfp4_gemm_impl(A, A_scales, K / 32, B, B_scales, K / 32, C, M, N, K, variant, stream);
}

extern "C" int hk_mxfp4_gemm(const void* A, const void* A_scales, const void* B, const void* B_scales,
                             void* C, int M, int N, int K, void* stream) {
    return mxfp4_gemm_impl(A, A_scales, K / 32, B, B_scales, K / 32, C, M, N, K, -1, stream);
}

extern "C" size_t hk_mxfp4_gemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0 || hk::gemm_dims_too_large(M, N, K)) return 0;
    const int s = hk::mxfp4_splitk_ranges(M, N, K);
    return s < 2 ? 0 : (size_t)s * M * N * sizeof(float);
}

extern "C" int hk_mxfp4_gemm_ws(const void* A, const void* A_scales, int a_scale_pitch, const void* B,
                                const void* B_scales, int b_scale_pitch, void* C, int M, int N, int K,
                                void* workspace, size_t workspace_bytes, void* stream) {
    using namespace hk;
    if (M <= 0 || N <= 0 || K <= 0 || (K % 32) != 0 || gemm_dims_too_large(M, N, K)) return HK_ERR_BAD_SHAPE;
    const int splits = mxfp4_splitk_ranges(M, N, K);
    // what the tile kernels need of the scale rows (see mxfp4_gemm_impl); anything else takes the plain path
    const Mxfp4ScaleRows sr = mxfp4_scale_rows(K, a_scale_pitch, b_scale_pitch);
    const bool tile_ok = sr.ok && A_scales && B_scales && (long long)(K / 2) * BM < (1ll << 31) &&
                         (long long)BM * max(a_scale_pitch, b_scale_pitch) < (1ll << 31);
    const bool can_split = splits >= 2 && workspace && workspace_bytes >= (size_t)splits * M * N * sizeof(float) &&
                           tile_ok && (long long)M * N < (1ll << 40);
    if (!can_split)
        return mxfp4_gemm_impl(A, A_scales, a_scale_pitch, B, B_scales, b_scale_pitch, C, M, N, K, -1, stream);
    if (!A || !B || !C) return HK_ERR_NULL_POINTER;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)workspace) & 15u) return HK_ERR_BAD_ALIGNMENT;
    // the skinny kernel adds its partial sums inside the workgroup and leaves the workspace alone
    if (use_skinny(M, N, (K / 2 + BK - 1) / BK, true, moe_num_compute_units(), kSkinnyMaxMScaled, 2))
        return mxfp4_gemm_impl(A, A_scales, a_scale_pitch, B, B_scales, b_scale_pitch, C, M, N, K, 6, stream);
    const bool edge = (M % kTinyTile) != 0 || (N % kTinyTile) != 0;
    return edge ? launch_mxfp4_splitk<true>(A, A_scales, B, B_scales, C, M, N, K, a_scale_pitch, b_scale_pitch, sr,
                                            splits, (float*)workspace, (hipStream_t)stream)
                : launch_mxfp4_splitk<false>(A, A_scales, B, B_scales, C, M, N, K, a_scale_pitch, b_scale_pitch, sr,
                                             splits, (float*)workspace, (hipStream_t)stream);
}

extern "C" int hk_mxfp4_gemm_pitched(const void* A, const void* A_scales, int a_scale_pitch, const void* B,
                                     const void* B_scales, int b_scale_pitch, void* C, int M, int N, int K,
                                     void* stream) {
    return mxfp4_gemm_impl(A, A_scales, a_scale_pitch, B, B_scales, b_scale_pitch, C, M, N, K, -1, stream);
}
