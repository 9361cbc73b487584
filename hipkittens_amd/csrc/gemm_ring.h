// The 4-wave GEMM schedule with a five-slot LDS ring, written once for every operand type whose
// K-step is 128 bytes per row (FP8: 128 elements, one MFMA per fragment pair; BF16: 64 elements, two).
#pragma once
#include "gemm_tile.h"

namespace hk {

// ---------------------------------------------------------------------------------------
// 4-wave schedule with a five-slot LDS ring (all 160 KiB): two slots for A tiles, three for B
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
//
// MMA is the operand type's policy:
//   Frag                          a wave's registers for 16 rows x 128 bytes of an operand
//   load(lo, hi, imm) -> Frag     from the two 16-byte LDS chunks of the lane's row
//   kPasses, mma<PASS>(acc, b, a) the MFMAs of one fragment pair (PASS 1.. are issued behind the
//                                 eight PASS 0 MFMAs of the same A fragment, so that two MFMAs
//                                 into one accumulator are eight issue slots apart)
//   raster_group(band_n, tiles_n) tile rows per raster group
// K: operand row pitch in bytes. `smem`: the workgroup's 160 KiB of LDS. STREAM_C: the epilogue's stores carry the
// non-temporal hint (store_c_tile).
template <typename MMA, bool EDGE, bool STREAM_C = false>
__device__ __forceinline__ void gemm_ring_body(uint8_t* smem, const uint8_t* __restrict__ A,
                                               const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
                                               int M, int N, int K, float alpha, int tiles_m, int tiles_n,
                                               int band_n) {
    using Frag = typename MMA::Frag;
    static_assert(MMA::kPasses == 1 || MMA::kPasses == 2, "the slot plan places at most two MFMAs per fragment pair");
    constexpr int NW = 4, TM = 128, TN = 128, MT = 8, NT = 8;
    constexpr int NDMA = kTileBytes / (NW * 1024);  // 8 loads per wave per operand per K-step
    constexpr int PG = 4, AD = 3;
    constexpr uint32_t kBRing = 2 * kTileBytes;      // B slots start behind the two A slots
    static_assert(PG == 4 && AD == 3 && MT == 8 && NDMA == 8, "slot plan below is written for these");

    const int lane = lane_id();
    const int w = wave_id();
    const int wm = w >> 1, wn = w & 1;

    int pm, pn;
    {
        const int id = xcd_chunk_order(blockIdx.x, tiles_m * tiles_n, kCuPerXcd);
        banded_raster(id, tiles_m, tiles_n, MMA::raster_group(band_n, tiles_n), band_n, pm, pn);
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
    Frag bf[2][NT];  // B fragments of the current / next K-step
    Frag af[4];      // rotating A fragments

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
    for (int n = 0; n < NT; ++n) bf[0][n] = MMA::load(b_lo0, b_hi0, n * 16 * BK);
#pragma unroll
    for (int m = 0; m < AD; ++m) af[m] = MMA::load(a_lo[0], a_hi[0], m * 16 * BK);

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
        // Two MFMAs per fragment pair (16-cycle MFMAs, each with room for about two other instructions, where
        // the 32-cycle FP8 MFMA has room for five): the operations behind the barrier are spread over the 48
        // MFMAs of both passes of groups 5..7 instead of the 24 of the first pass (+1.5 % for BF16 at 8192^3).
        // Slot q (0..47) = 16 (m - 5) + 8 pass + n: LDS reads in the even slots, unit q / 2 = B0..B7, A0, A1,
        // then A2 at q = 32 (A fragment j's registers are free once group 4 + j is done, i.e. from q = 16 j
        // on); the eight A loads at q = 1, 5, .., 29. (Splitting a load into its M0 write and the load itself,
        // one slot apart, which also saves the wait state between them, measured the same.)
        auto post_ops = [&](int q) __attribute__((always_inline)) {
            if ((q & 1) == 0) {
                const int u = q / 2;
                if (u < NT) bf[P ^ 1][u] = MMA::load(bl, bh, u * 16 * BK);
                else if (u == NT || u == NT + 1) af[u - NT] = MMA::load(a_lo[P ^ 1], a_hi[P ^ 1], (u - NT) * 16 * BK);
                else if (u == 16) af[2] = MMA::load(a_lo[P ^ 1], a_hi[P ^ 1], 2 * 16 * BK);
            } else if (q % 4 == 1 && q / 4 < NDMA) {
                dma_a(q / 4, P, k2, sa, vor);
            }
        };
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                MMA::template mma<0>(acc[m][n], bf[P][n], af[m & 3]);
                if (m <= PG) {
                    const int s = m * NT + n;  // 40 slots before the barrier: B loads at 2, 7, .., 37
                    if (n == 0) af[(m + AD) & 3] = MMA::load(a_lo[P], a_hi[P], (m + AD) * 16 * BK);
                    if (s % 5 == 2) dma_b(s / 5, off2, k2, sb, vor);
                } else if (MMA::kPasses == 2) {
                    post_ops((m - PG - 1) * 16 + n);
                } else {
                    const int j = (m - PG - 1) * NT + n;  // 24 slots after the barrier
                    if (j < NT) {
                        bf[P ^ 1][j] = MMA::load(bl, bh, j * 16 * BK);
                    } else if (j == NT || j == NT + 1) {
                        af[j - NT] = MMA::load(a_lo[P ^ 1], a_hi[P ^ 1], (j - NT) * 16 * BK);
                    } else if (j == 2 * NT) {
                        af[2] = MMA::load(a_lo[P ^ 1], a_hi[P ^ 1], 2 * 16 * BK);
                    }
                    if (j < 2 * NDMA && (j & 1)) dma_a(j >> 1, P, k2, sa, vor);  // A loads at 1, 3, .., 15
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int pass = 1; pass < MMA::kPasses; ++pass)
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    MMA::template mma<1>(acc[m][n], bf[P][n], af[m & 3]);
                    if (m > PG) post_ops((m - PG - 1) * 16 + 8 + n);
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

    store_c_tile<MT, NT, EDGE, STREAM_C>(acc, C, M, N, row0 + wm * TM, col0 + wn * TN, alpha);
}

}  // namespace hk
