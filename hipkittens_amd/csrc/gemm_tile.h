// Pieces shared by the 256x256 tile GEMM kernels (FP8 and MXFP4): tile geometry, the
// column permutation of the B tile and the bf16 epilogue.
#pragma once
#include "hk_device.h"

namespace hk {

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kTileBytes = BM * BK;           // one operand tile in LDS (32 KiB)
constexpr int kStageBytes = 2 * kTileBytes;   // A tile + B tile
constexpr int kLdsBytes = 2 * kStageBytes;    // two stages (128 KiB)

// Width of the raster's column bands in tiles (banded_raster): operands that fit the 256 MB
// memory-side cache together are walked in stripes across all tile columns; larger ones in bands of
// 16 tile columns, so that a band's B panels stay cached while its A rows stream past. Measured:
// +4 to 5 % at 16384^3 for FP8 (512 MB of operands) and BF16 (1 GB), -0.5 % at 256 MB and below and
// -4 % for MXFP4 at 16384^3 (256 MB), hence the threshold.
inline int raster_band(long long operand_bytes, int tiles_n) {
    return operand_bytes > (320ll << 20) ? 16 : tiles_n;
}

// Position of LDS row R of the B tile inside the tile's 256 columns of C:
// within each group of 32 rows, row 16*t + r (t = MFMA tile parity, r = operand
// row) holds column 8*(r/4) + 4*t + r%4.
__device__ __forceinline__ int b_row_to_col(int R) {
    const int r = R & 15, t = (R >> 4) & 1;
    return (R & ~31) | ((r >> 2) << 3) | (t << 2) | (r & 3);
}

// The two 16-byte halves of a lane's fragment row (chunks g and g + 4 of the 128-byte row) as
// separate operands, for kernels whose MFMA consumes 16 bytes per lane: MXFP4 (MX blocks g and
// 4 + g of a 256-element K-step) and bf16 (elements 8g.. and 32 + 8g.. of a 64-element K-step).
struct Frag4 {
    v4i lo, hi;
};
__device__ __forceinline__ Frag4 lds_frag4(uint32_t addr_lo, uint32_t addr_hi, int imm) {
    Frag4 f;
    f.lo = *(lds_v4i_t*)(uintptr_t)(addr_lo + imm);
    f.hi = *(lds_v4i_t*)(uintptr_t)(addr_hi + imm);
    return f;
}

// Epilogue of the tile kernels: alpha, bf16 (RNE), 16-byte stores.
// acc[m][2p], acc[m][2p+1] hold, for C row `row_base + 16m + lane%16`, the 8 columns
// `col_base + 32p + 8*(lane/16) .. +8` (see b_row_to_col).
// STREAM: the full-tile stores carry the non-temporal hint (C is written once and not read by the kernel;
// keeping it out of the L2 leaves that cache to the operand panels). Only the BF16 ring kernel has an
// instantiation with it (bf16_gemm.hip has the measurements).
template <int MT, int NT, bool EDGE, bool STREAM = false>
__device__ __forceinline__ void store_c_tile(const v4f (&acc)[MT][NT], uint16_t* __restrict__ C,
                                             int M, int N, int row_base, int col_base, float alpha) {
    const int r = lane_id() & 15, g = lane_id() >> 4;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int row = row_base + 16 * m + r;
#pragma unroll
        for (int p = 0; p < NT / 2; ++p) {
            const int col = col_base + 32 * p + 8 * g;
            const v4f x = acc[m][2 * p] * alpha, y = acc[m][2 * p + 1] * alpha;
            if (!EDGE) {
                v4i out;
                out.x = pack_bf16(x.x, x.y); out.y = pack_bf16(x.z, x.w);
                out.z = pack_bf16(y.x, y.y); out.w = pack_bf16(y.z, y.w);
                if (STREAM) __builtin_nontemporal_store(out, (v4i*)(C + (size_t)row * N + col));
                else *(v4i*)(C + (size_t)row * N + col) = out;
            } else if (row < M) {
                const float v[8] = {x.x, x.y, x.z, x.w, y.x, y.y, y.z, y.w};
                if (col + 8 <= N && (N & 7) == 0) {
                    v4i out;
                    out.x = pack_bf16(v[0], v[1]); out.y = pack_bf16(v[2], v[3]);
                    out.z = pack_bf16(v[4], v[5]); out.w = pack_bf16(v[6], v[7]);
                    *(v4i*)(C + (size_t)row * N + col) = out;
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (col + j < N)
                            C[(size_t)row * N + col + j] = (uint16_t)(pack_bf16(v[j], 0.f) & 0xffffu);
                }
            }
        }
    }
}

}  // namespace hk
