// MXFP4 fused MoE for gfx950: activation quantization, grouped gate+up GEMM with SiLU-mul and
// MX re-quantization in the epilogue, grouped down GEMM, weighted un-permute.
//
// The reference has no MoE code (no counterpart to cite); the GEMM core follows the 4-wave
// interleaved FP8/MXFP4 kernels of this library (LDS-direct loads into swizzled 128-byte-row
// tiles, ds_read_b128 fragments, v_mfma_scale_f32_16x16x128_f8f6f4 with in-MFMA e8m0 scales).
//
// Grouped GEMM: a work item is (m-tile, n-tile) where an m-tile is a run of consecutive rows
// (sorted positions) of one expert; the item list is built on the device from expert_offsets.
// Weights dominate HBM traffic, so workgroups are persistent (one per CU) and keep their operand
// pipelines running across item boundaries. Items that share an expert run at the same time on
// the CUs of one XCD, so activation tiles come out of that XCD's L2 and every weight byte leaves
// HBM once. Two kernels: moe_mxfp4_stream4_kernel for weights in the pre-shuffled layout (the fast
// path: weights go straight from HBM into MFMA operand registers, 192-row m-tiles) and
// moe_mxfp4_gemm_kernel for the plain layout (both operands through an LDS ring, 128-row m-tiles).
#include "moe_common.h"
#include "moe_sort.h"
#include "../../include/hk355.h"

namespace hk {

typedef __attribute__((address_space(3))) const v2i lds_v2i_t;

// ------------------------------------------------------------------------ MX quantization
// e8m0 exponent for a block with maximum magnitude amax: floor(log2(amax)) - 2, clamped to
// [-127, 127]; 0 for an all-zero block.
__device__ __forceinline__ int mx_block_exponent(float amax) {
    if (!(amax > 0.f)) return 0;
    const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127 - 2;
    return max(-127, min(127, e));
}
// Eight values times 2^-e as packed e2m1 codes (round to nearest, ties to the even code,
// saturating at 6; element i in nibble i). v_cvt_scalef32_pk_fp4_f32 divides by the power-of-two
// scale and rounds exactly like that, NaN and infinities included (checked against the compare
// chain of the CPU oracle over all bf16 inputs, the ties and their neighbours, e = -127..127).
__device__ __forceinline__ uint32_t pack8_e2m1(const float (&v)[8], int e) {
    // 2^e as a float; 2^-127 is the denormal 0x00400000
    const float scale = __uint_as_float(e > -127 ? (uint32_t)(e + 127) << 23 : 0x00400000u);
    uint32_t out = 0;
    out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[0], v[1], scale, 0);
    out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[2], v[3], scale, 1);
    out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[4], v[5], scale, 2);
    out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[6], v[7], scale, 3);
    return out;
}
// MXFP8 (e4m3 elements): shared exponent floor(log2(amax)) - 8, clamped to [-127, 127]; 0 for an
// all-zero block.
__device__ __forceinline__ int mx8_block_exponent(float amax) {
    if (!(amax > 0.f)) return 0;
    const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127 - 8;
    return max(-127, min(127, e));
}
// Eight values times 2^-e as e4m3 codes (round to nearest even), saturating at +-448: the values
// are clamped to +-448 * 2^e first (a block maximum in [1.75, 2) * 2^(e + 8) lies above), the
// conversion divides by the power-of-two scale exactly. Element i in byte i.
__device__ __forceinline__ v2i pack8_e4m3(const float (&v)[8], int e) {
    typedef short v2s __attribute__((ext_vector_type(2)));
    const float scale = __uint_as_float(e > -127 ? (uint32_t)(e + 127) << 23 : 0x00400000u);
    // 448 * 2^e = 1.75 * 2^(e + 8); beyond the float range there is nothing to clamp
    const float lim = __uint_as_float(e + 8 + 127 < 255 ? ((uint32_t)(e + 8 + 127) << 23) | 0x00600000u : 0x7f7fffffu);
    float c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = __builtin_amdgcn_fmed3f(v[i], -lim, lim);
    v2s lo = {0, 0}, hi = {0, 0};
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(lo, c[0], c[1], scale, false);
    lo = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(lo, c[2], c[3], scale, true);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(hi, c[4], c[5], scale, false);
    hi = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(hi, c[6], c[7], scale, true);
    return v2i{__builtin_bit_cast(int, lo), __builtin_bit_cast(int, hi)};
}
// Gated activation of the extended epilogues. act 0: SiLU(g) * u; act 1: the clamped SwiGLU of
// the GPT-OSS experts, (clamp(u, -limit, limit) + 1) * g' * sigmoid(alpha * g') with
// g' = min(g, limit).
__device__ __forceinline__ float glu_act(int act, float g, float u, float alpha, float limit) {
    if (act == 0) return silu_mul(g, u);
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return (u + 1.0f) * (g * __builtin_amdgcn_rcpf(1.0f + __expf(-alpha * g)));
}

// x [rows, cols] bf16 -> packed e2m1 [rows, cols/2] + e8m0 scales [rows, scale_pitch] (columns
// >= cols/32 are filled with 127). One thread per 8 elements, 4 threads per MX block.
template <bool A8>
__global__ __launch_bounds__(256) void mx_quantize_rows_kernel(const uint16_t* __restrict__ x, int rows,
                                                               int cols, uint8_t* __restrict__ packed,
                                                               uint8_t* __restrict__ scales,
                                                               int scale_pitch) {
    const int per_row = scale_pitch * 4;  // threads per row, a multiple of 4 (and of 32: pitch % 8 == 0)
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const int row = (int)(gid / per_row);
    const int c8 = (int)(gid % per_row);  // which group of 8 elements
    if (row >= rows) return;
    float v[8];
    const bool in = c8 * 8 < cols;
    if (in) {
        const v4i raw = *(const v4i*)(x + (size_t)row * cols + c8 * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float((uint32_t)raw[i] << 16);
            v[2 * i + 1] = __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = 0.f;
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    const int e = A8 ? mx8_block_exponent(amax) : mx_block_exponent(amax);
    if (in) {
        if (A8) *(v2i*)(packed + (size_t)row * cols + c8 * 8) = pack8_e4m3(v, e);
        else *(uint32_t*)(packed + (size_t)row * (cols / 2) + c8 * 4) = pack8_e2m1(v, e);
    }
    if ((c8 & 3) == 0) scales[(size_t)row * scale_pitch + (c8 >> 2)] = (uint8_t)(e + 127);
}

// Item lists of the two grouped GEMMs of a layer: list `which` (0 / 1) covers n_tiles[which] tiles
// of weight rows and goes to items[which], its length to num_items[which]. One workgroup of NT
// threads per list; thread t owns experts [t * 512 / NT, (t + 1) * 512 / NT). `scan`: NT ints of LDS.
// With nparts > 1 workgroups per list, workgroup `part` writes the n-tiles part, part + nparts, ...
struct MoeBuildItems { MoeItem* items[2]; int n_tiles[2]; int bm; };
// moe_build_items_ranges: the same from the experts' row ranges [lo[j], hi[j]) held by the threads
// (thread t: experts t * 512 / NT + j).
template <int NT>
__device__ __forceinline__ void moe_build_items_ranges(const int (&lo)[512 / NT], const int (&hi)[512 / NT], int E,
                                                       const MoeBuildItems& b, int which,
                                                       int32_t* __restrict__ num_items, int* scan,
                                                       int part = 0, int nparts = 1) {
    constexpr int EPT = 512 / NT;
    const int n_tiles_n = b.n_tiles[which], bm = b.bm;
    MoeItem* __restrict__ items = b.items[which];
    const int t = threadIdx.x;
    int cnt[EPT], mine = 0;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        cnt[j] = t * EPT + j < E ? (hi[j] - lo[j] + bm - 1) / bm : 0;
        mine += cnt[j] * n_tiles_n;
    }
    scan[t] = mine;
    __syncthreads();
    for (int d = 1; d < NT; d <<= 1) {
        const int v = t >= d ? scan[t - d] : 0;
        __syncthreads();
        scan[t] += v;
        __syncthreads();
    }
    int base = scan[t] - mine;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        // an expert's rows are spread evenly over its items (in whole 16-row fragments): items of one
        // expert then take the same time, run side by side and share the expert's weights in L2
        const int R = hi[j] - lo[j];
        int per = cnt[j] > 0 ? ((R + cnt[j] - 1) / cnt[j] + 15) & ~15 : bm;
        if (per > bm || (cnt[j] - 1) * per >= R) per = bm;
        for (int n = part; n < n_tiles_n; n += nparts)
            for (int m = 0; m < cnt[j]; ++m) {
                MoeItem it;
                it.expert = t * EPT + j; it.row_start = lo[j] + m * per; it.rows = min(per, hi[j] - it.row_start);
                it.n_tile = n;
                items[base + n * cnt[j] + m] = it;
            }
        base += cnt[j] * n_tiles_n;
    }
    if (t == NT - 1 && part == 0) num_items[which] = scan[NT - 1];
}
template <int NT>
__device__ __forceinline__ void moe_build_items_block(const int32_t* __restrict__ expert_offsets, int E,
                                                      const MoeBuildItems& b, int which,
                                                      int32_t* __restrict__ num_items, int* scan,
                                                      int part = 0, int nparts = 1) {
    constexpr int EPT = 512 / NT;
    int lo[EPT], hi[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        const int e = threadIdx.x * EPT + j;
        lo[j] = e < E ? expert_offsets[e] : 0;
        hi[j] = e < E ? expert_offsets[e + 1] : 0;
    }
    moe_build_items_ranges<NT>(lo, hi, E, b, which, num_items, scan, part, nparts);
}

__global__ __launch_bounds__(512) void moe_build_items_kernel(const int32_t* __restrict__ expert_offsets,
                                                              int E, MoeBuildItems b,
                                                              int32_t* __restrict__ num_items) {
    __shared__ int scan[512];
    moe_build_items_block<512>(expert_offsets, E, b, blockIdx.x, num_items, scan, blockIdx.y, gridDim.y);
}

// Activation layout inside the MoE ("K-step-major tiles"): for a matrix of S rows the bytes of
// K-step kt (256 elements = 128 bytes per row, zero-padded past K) of all rows are contiguous,
//   data   [nk][S][128] bytes,   scales [nk][S][8] e8m0 bytes (padding = 127),
// so that the A tile of a work item (consecutive rows) and its scale tile are single contiguous,
// 128-byte aligned runs for the global->LDS loads.
//
// Quantize-and-permute: row `pos` of the output is token sorted_slots[pos] / topk of x, so that
// each expert's rows are contiguous for the grouped GEMM (the "permute" step of the MoE). The
// kernel walks tokens, not output rows: a row of x is read and quantized once and stored to the
// positions of the token's topk slots (slot_to_pos), instead of being fetched once per slot.
// A slot's position is used only if sorted_slots maps it back to the slot (slots that took no
// part in the sort have no position).
// The same launch pads the second tiled matrix of the layer (h, contraction length K2): the part
// of its last K-step past K2 that the producing GEMM epilogue never writes is set to zero data
// and neutral scales (nothing to do when K2 is a multiple of 256).
// Launch: 128 threads = 4 K-steps x 32 threads (8 elements each) for kQpRows tokens; grid
// (ceil(T / kQpRows) + 2, ceil(nk / 4)).
// The two columns of workgroups past the tokens build the layer's two work-item lists instead (the
// gridDim.y workgroups of a column share a list's n-tiles), which need only expert_offsets and so
// ride along in the shadow of the quantization.
// A8: MXFP8 activations (e4m3 elements): 256 bytes per row and K-step in both tiled matrices.
// PERMUTE false: no permutation, one output row per token (data [nk][T][..]; the 4-wave streaming
// kernel gathers its rows by token and needs neither the topk copies of a row nor the sort's result
// here: sorted_slots / slot_to_pos are not read), and the scales of 16 K-steps share a 128-byte row:
// scales [ceil(nk / 16)][T][128], K-step kt at byte 8 (kt % 16) of the row of super-step kt / 16.
constexpr int kQpRows = 4;   // tokens per workgroup
struct MxQuantizeArgs {
    const uint16_t* x; const int32_t* sorted_slots; const int32_t* slot_to_pos;
    int topk, T, cols;
    uint8_t* tiled; uint8_t* tiled_scales; uint8_t* tiled2; uint8_t* tiled2_scales;
    int K2;
};
// The work of 32 threads (c = 0..31: 8 elements each) on K-step kt of tokens t0 .. t0 + kQpRows - 1;
// `pad` set for one group of 32 threads per token block: it also pads the second matrix.
template <bool A8, bool PERMUTE>
__device__ __forceinline__ void mx_quantize_tokens(const MxQuantizeArgs& a, int t0, int kt, int c, bool pad) {
    const int T = a.T, topk = a.topk, cols = a.cols, K2 = a.K2;
    const uint16_t* __restrict__ x = a.x;
    const int32_t* __restrict__ sorted_slots = a.sorted_slots;
    const int32_t* __restrict__ slot_to_pos = a.slot_to_pos;
    uint8_t* __restrict__ tiled = a.tiled;
    uint8_t* __restrict__ tiled_scales = a.tiled_scales;
    uint8_t* __restrict__ tiled2 = a.tiled2;
    uint8_t* __restrict__ tiled2_scales = a.tiled2_scales;
    const int S = T * topk;
    const int nk = (cols / 2 + 127) >> 7;
    // position of slot `slot`, or -1
    auto position = [&](int slot) -> int {
        if (!PERMUTE) return slot;
        const int pos = slot_to_pos[slot];
        return (unsigned)pos < (unsigned)S && sorted_slots[pos] == slot ? pos : -1;
    };
    if (pad && (K2 & 255)) {
        const int nk2 = (K2 + 255) >> 8;
        const int valid = K2 - (nk2 - 1) * 256;  // valid elements of the last K-step, a multiple of 32
        for (int j = 0; j < kQpRows && t0 + j < T; ++j)
            for (int q = 0; q < topk; ++q) {
                const int pos = position((t0 + j) * topk + q);
                if (pos < 0) continue;
                const size_t tile_row2 = (size_t)(nk2 - 1) * S + pos;
                if (c * 8 >= valid) {
                    if (A8) *(v2i*)(tiled2 + tile_row2 * 256 + c * 8) = v2i{0, 0};
                    else *(uint32_t*)(tiled2 + tile_row2 * 128 + c * 4) = 0u;
                }
                if (c < 8 && c * 32 >= valid) tiled2_scales[tile_row2 * 8 + c] = 127;
            }
    }
    if (kt >= nk) return;
    const int col = kt * 256 + c * 8;
    // the loads of the workgroup's rows are issued together: a thread's 16 bytes per row are all it has in flight
    v4i raw[kQpRows];
#pragma unroll
    for (int j = 0; j < kQpRows; ++j)
        raw[j] = col < cols ? *(const v4i*)(x + (size_t)min(t0 + j, T - 1) * cols + col) : v4i{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < kQpRows; ++j) {
        if (t0 + j >= T) break;
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float((uint32_t)raw[j][i] << 16);
            v[2 * i + 1] = __uint_as_float((uint32_t)raw[j][i] & 0xffff0000u);
        }
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        const int e = A8 ? mx8_block_exponent(amax) : mx_block_exponent(amax);
        v2i q8 = {0, 0};
        uint32_t q4 = 0;
        if (A8) q8 = pack8_e4m3(v, e);
        else q4 = pack8_e2m1(v, e);
        for (int q = 0; q < (PERMUTE ? topk : 1); ++q) {
            const int pos = PERMUTE ? position((t0 + j) * topk + q) : t0 + j;
            if (pos < 0) continue;
            const size_t tile_row = (size_t)kt * (PERMUTE ? S : T) + pos;
            if (A8) *(v2i*)(tiled + tile_row * 256 + c * 8) = q8;
            else *(uint32_t*)(tiled + tile_row * 128 + c * 4) = q4;
            if ((c & 3) == 0) {
                if (PERMUTE) tiled_scales[tile_row * 8 + (c >> 2)] = (uint8_t)(e + 127);
                else tiled_scales[((size_t)(kt >> 4) * T + pos) * 128 + (kt & 15) * 8 + (c >> 2)] = (uint8_t)(e + 127);
            }
        }
    }
}

template <bool A8, bool PERMUTE>
__global__ __launch_bounds__(128) void mx_quantize_permute_kernel(MxQuantizeArgs a,
                                                                  const int32_t* __restrict__ expert_offsets, int E,
                                                                  MoeBuildItems items, int32_t* __restrict__ num_items) {
    __shared__ int scan[128];
    const int tok_blocks = (a.T + kQpRows - 1) / kQpRows;
    if ((int)blockIdx.x >= tok_blocks) {
        // list blockIdx.x - tok_blocks, its n-tiles shared by the gridDim.y workgroups of this column
        moe_build_items_block<128>(expert_offsets, E, items, (int)blockIdx.x - tok_blocks, num_items, scan,
                                   blockIdx.y, gridDim.y);
        return;
    }
    mx_quantize_tokens<A8, PERMUTE>(a, blockIdx.x * kQpRows, blockIdx.y * 4 + (threadIdx.x >> 5), threadIdx.x & 31,
                                    blockIdx.y == 0 && threadIdx.x < 32);
}

// One launch for a layer of at most kSortSmallMax slots whose gate+up kernel gathers its rows by
// token: the sort of the slots (moe_sort_small_block, workgroups [0, nchunks)), the layer's two
// work-item lists (2 * kFusedItemParts workgroups: each repeats the sort's histogram and scan, which
// gives it the experts' row ranges without waiting for anyone, and writes a share of one list) and
// the quantization of x (the remaining workgroups: 8 K-steps x 32 threads for kQpRows tokens), which
// needs nothing from the sort. The quantization then costs the layer no time of its own.
constexpr int kFusedItemParts = 4;
template <bool A8>
__global__ __launch_bounds__(256) void moe_sort_quantize_kernel(const int32_t* __restrict__ ids, int E,
                                                                int32_t* __restrict__ expert_offsets,
                                                                int32_t* __restrict__ sorted_slots,
                                                                int32_t* __restrict__ slot_to_pos, MxQuantizeArgs a,
                                                                MoeBuildItems items, int32_t* __restrict__ num_items) {
    __shared__ MoeSortSmallLds lds;
    const int S = a.T * a.topk;
    const int nchunks = (S + kSortChunk - 1) / kSortChunk;
    int b = blockIdx.x;
    int lo[2], hi[2];
    if (b < nchunks) {
        moe_sort_small_block(ids, S, E, b, true, expert_offsets, sorted_slots, slot_to_pos, lds, lo, hi);
        return;
    }
    b -= nchunks;
    if (b < 2 * kFusedItemParts) {
        moe_sort_small_block(ids, S, E, nchunks, false, expert_offsets, sorted_slots, slot_to_pos, lds, lo, hi);
        __syncthreads();   // the scan array below reuses the sort's LDS
        moe_build_items_ranges<256>(lo, hi, E, items, b / kFusedItemParts, num_items, &lds.round_cnt[0][0],
                                    b % kFusedItemParts, kFusedItemParts);
        return;
    }
    b -= 2 * kFusedItemParts;
    const int nk = (a.cols / 2 + 127) >> 7, kgroups = (nk + 7) / 8;
    const int kg = b % kgroups;
    mx_quantize_tokens<A8, false>(a, (b / kgroups) * kQpRows, kg * 8 + (threadIdx.x >> 5), threadIdx.x & 31,
                                  kg == 0 && threadIdx.x < 32);
}

// ---------------------------------------------------------------------- weight pre-shuffle
// Tile row R (0..255) of n-tile `n_tile` in the pre-shuffled layout -> row of the expert's weight
// matrix. The layout is written in units of 32 tile rows (`w` below, two MFMA fragments); wave W of
// moe_mxfp4_stream4_kernel owns units 2 W and 2 W + 1, i.e. tile rows [64 W, +64).
// mode 0 (gate+up, N = I): fragment 0 holds the gate rows and fragment 1 the up rows of h columns
// 128 n_tile + 16 w .. +16, in order; mode 1 (down, N = H): the b_row_to_col permutation, which
// gives a lane 8 consecutive output columns from its two fragments. Rows past N repeat row N - 1.
// mode 2: as mode 0 for a source matrix with gate / up of h column c in rows 2c / 2c + 1.
__device__ __forceinline__ int moe_stream_b_row(int mode, int R, int n_tile, int N) {
    if (mode == 1) return min(n_tile * 256 + b_row_to_col(R), N - 1);
    const int w = R >> 5, f = (R >> 4) & 1, r = R & 15;
    const int hcol = min(n_tile * 128 + 16 * w + r, N - 1);
    return mode == 2 ? 2 * hcol + f : f * N + hcol;
}

// Pre-shuffled weight layout, made for moe_mxfp4_stream4_kernel: weights go from HBM straight
// into MFMA operand registers, so for every (expert, n-tile of 256 tile rows, K-step of 256
// elements) one contiguous 32 KiB block holds, unit by unit (unit w = tile rows [32 w, +32)),
// the unit's four B fragments f = 2 * nfrag + half as 1 KiB pieces in lane order: lane l's 16
// bytes are tile row 32 w + 16 nfrag + l % 16 (moe_stream_b_row gives the weight row), K bytes
// 128 kt + 64 half + 16 (l / 16) .. +16, zero past the end of K. A second array holds the
// scales the same way, 4 bytes per lane: byte 2 half + nfrag is the e8m0 scale of that row's
// 32-element block 8 kt + 4 half + l / 16 (127 past the end of K).
//   out_w [E][n_tiles][nk][8][4][64][16] bytes, out_s [E][n_tiles][nk][8][64][4] bytes.
__global__ __launch_bounds__(256) void moe_preshuffle_kernel(const uint8_t* __restrict__ w,
                                                             const uint8_t* __restrict__ sc, int E, int N,
                                                             int K, int scale_pitch, int mode, int n_tiles,
                                                             uint8_t* __restrict__ out_w,
                                                             uint8_t* __restrict__ out_s) {
    const int Kb = K >> 1, nk = (Kb + 127) >> 7;
    const int rows_b = mode == 1 ? N : 2 * N;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;  // one 16-byte chunk each
    const long long total = (long long)E * n_tiles * nk * 2048;
    if (gid >= total) return;
    const int l = (int)(gid & 63), f = (int)((gid >> 6) & 3), wv = (int)((gid >> 8) & 7);
    long long rest = gid >> 11;
    const int kt = (int)(rest % nk); rest /= nk;
    const int nt = (int)(rest % n_tiles);
    const int e = (int)(rest / n_tiles);
    const int row = moe_stream_b_row(mode, 32 * wv + 16 * (f >> 1) + (l & 15), nt, N);
    const int kb = kt * 128 + 64 * (f & 1) + 16 * (l >> 4);
    v4i val = {0, 0, 0, 0};
    if (kb < Kb) val = *(const v4i*)(w + ((size_t)e * rows_b + row) * Kb + kb);
    *(v4i*)(out_w + gid * 16) = val;
    if (f == 0) {
        // this thread also writes the lane's 4 scale bytes of the K-step
        uint8_t* dst = out_s + ((gid >> 11) * 8 + wv) * 256 + l * 4;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int rw = moe_stream_b_row(mode, 32 * wv + 16 * (b & 1) + (l & 15), nt, N);
            const int blk = kt * 8 + 4 * (b >> 1) + (l >> 4);
            dst[b] = blk < (K >> 5) ? sc[((size_t)e * rows_b + rw) * scale_pitch + blk] : (uint8_t)127;
        }
    }
}

// ---------------------------------------------------------------------------- grouped GEMM
struct MoeGemmParams {
    const uint8_t* A;        // activations in sorted order, K-step-major tiles [nk][S][128]
    const uint8_t* SA;       // their e8m0 scales [nk][S][8]
    const uint8_t* B;        // expert weights, packed e2m1 [E][rows_b][b_pitch]
    const uint8_t* SB;       // their scales [E][rows_b][sb_pitch]
    const MoeItem* items;
    const int32_t* num_items;
    void* out0;              // MODE 0: packed h as K-step-major tiles [nk2][S][128]; MODE 1: bf16 o [S][N]
    uint8_t* out_scales;     // MODE 0: e8m0 scales of h [nk2][S][8]
    long long b_expert_stride, sb_expert_stride;
    int b_pitch, sb_pitch;   // plain weight layout only
    int S;                   // rows of the activation matrices (T * topk)
    // Gathered activations (the 4-wave streaming kernel, MODE 0): A / SA hold one row per TOKEN
    // ([nk][a_rows][..], a_rows = T) and sorted row `pos` of the GEMM is token row_slots[pos] / topk.
    const int32_t* row_slots;
    int a_rows;
    uint32_t topk_magic;     // ceil(2^32 / topk), or 0 for topk == 1: slot / topk = umulhi(slot, magic) for slot < 2^24
    int K;                   // contraction length in elements
    int N;                   // MODE 0: I (h columns; weight rows i and I+i); MODE 1: output columns
    int n_tiles_n;
    // extended epilogues (kernels instantiated with EXT) only:
    const float* bias;       // null or fp32 [E][rows of B] in the caller's row order, added to the GEMM result
    uint32_t bias_bytes;     // size of that array (the streaming kernel reads it through a range-checked descriptor)
    int act;                 // MODE 0: 0 = SiLU(gate) * up, 1 = clamped SwiGLU (glu_act)
    float alpha, limit;
    int interleaved;         // MODE 0: the caller's gate / up rows (and biases) of h column c are 2c / 2c + 1
};

constexpr int kMoeATile = kMoeBM * 128;                 // 16 KiB
constexpr int kMoeBTile = 256 * 128;                    // 32 KiB
constexpr int kMoeStage = kMoeATile + kMoeBTile;        // 64 KiB
constexpr int kMoeStages = 3;
constexpr int kMoeScaleA = kMoeBM * 8, kMoeScaleB = 256 * 8;
constexpr int kMoeScaleStage = kMoeScaleA + kMoeScaleB; // 4 KiB
constexpr int kMoeScaleBase = kMoeStages * kMoeStage;
constexpr int kMoeLds = kMoeScaleBase + kMoeStages * kMoeScaleStage;  // 153 KiB

// Global->LDS source offsets of one work item.
struct MoeAddr {
    v4i srd_b, srd_sb;
    uint32_t voff_b[4], voff_sb;
    int row_start, rows, n0, n_tile, expert;
    bool valid;
};

// 8 waves (two per SIMD), wave (wm, wn) = (w / 4, w % 4) owns the 16-row fragments 2m + wm
// (m = 0..7: even or odd fragments, so that both waves of a SIMD have work whatever the tile's
// row count) x weight rows [64 wn, +64) of the 256 x 256 tile. The K loop is deliberately simple - wait for the K-step's
// operands, one barrier, start the loads of the next K-step into the other LDS stage, compute -
// because the two waves of a SIMD cover for each other: while one is held up issuing loads or
// waiting for LDS, the other feeds the matrix pipe (a single wave per SIMD cannot issue the
// 16-cycle FP4 MFMA back to back, nor issue loads and MFMAs at the same time).
template <int MODE, bool EXT>
__global__ __launch_bounds__(512) void moe_mxfp4_gemm_kernel(const MoeGemmParams p) {
    constexpr int NW = 8, MT = kMoeBM / 32, NT = 4;   // MT fragments of 16 rows per wave
    constexpr int NA = kMoeBM / 64;                  // A-tile loads per wave and K-step
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    const int lane = lane_id(), w = wave_id();
    const int wm = w >> 2, wn = w & 3;
    // Item assignment. Workgroup ids go round robin over the 8 XCDs; each XCD takes a contiguous
    // range of the item list and its workgroups walk that range with a stride equal to their
    // number, so that at any time the CUs of one XCD work on consecutive items = the same
    // expert's rows with neighbouring n-tiles, and share that expert's activation tile in the
    // XCD's L2 (each weight tile is needed exactly once anyway).
    const int n_items = scalar_load_x1(p.num_items);
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int it_stride = ((int)gridDim.x - xcd + kNumXcd - 1) / kNumXcd;  // workgroups on this XCD
    const int per_xcd = (n_items + kNumXcd - 1) / kNumXcd;
    int it = xcd * per_xcd + slot;
    const int it_end = min(n_items, (xcd + 1) * per_xcd);
    if (it >= it_end) return;

    const int Kb = p.K >> 1;                 // contraction bytes per row
    const int nk = (Kb + 127) >> 7;
    const int tail_bytes = Kb - (nk - 1) * 128;  // valid bytes of the last K-step (16..128)
    const int rows_b = MODE == 0 ? 2 * p.N : p.N;
    // loads per wave and K-step: A tile, B tile, A scales, B scales
    constexpr int kDma = NA + 4 + 2;
    const v4i srd_a = make_srd(p.A, (uint32_t)nk * (uint32_t)p.S * 128u);
    const v4i srd_sa = make_srd(p.SA, (uint32_t)nk * (uint32_t)p.S * 8u);

    // Load i of this wave fills LDS rows 8*(i*NW + w) .. +8 of a tile; lane l lands in row +l/8,
    // physical chunk l%8 and fetches logical chunk swz(row, l%8), the same for every i.
    const uint32_t chunk16 = swz_chunk(8 * w + (lane >> 3), lane & 7);
    const bool tail_oob = (int)(chunk16 * 16) >= tail_bytes;

    auto make_addr = [&](int idx, MoeAddr& a) {
        a.valid = idx < it_end;
        if (!a.valid) idx = it_end - 1;  // harmless values; every load of an invalid set is zero-sized
        const v4i item = scalar_load_x4(p.items + idx);  // {expert, row_start, rows, n_tile}
        const int expert = item.x;
        a.expert = expert;
        a.row_start = item.y;
        a.rows = item.z;
        a.n_tile = item.w;
        a.n0 = a.n_tile * (MODE == 0 ? 128 : 256);
        a.srd_b = make_srd(p.B + (size_t)expert * p.b_expert_stride, (uint32_t)rows_b * (uint32_t)p.b_pitch);
        a.srd_sb = make_srd(p.SB + (size_t)expert * p.sb_expert_stride, (uint32_t)rows_b * (uint32_t)p.sb_pitch);
        auto b_row = [&](int R) -> int { return moe_b_row(MODE, R, a.n_tile, p.N, EXT && p.interleaved); };
#pragma unroll
        for (int i = 0; i < 4; ++i)
            a.voff_b[i] = (uint32_t)b_row(8 * (i * NW + w) + (lane >> 3)) * (uint32_t)p.b_pitch + chunk16 * 16u;
        a.voff_sb = (uint32_t)b_row(32 * w + (lane >> 1)) * (uint32_t)p.sb_pitch + (lane & 1) * 4u;
    };

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    // scale pieces per wave: A scales of kMoeBM/8 rows and B scales of 32 rows
    const uint32_t sa_bytes = kMoeBM;  // A-scale bytes per loading wave
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kMoeScaleBase + (uint32_t)w * sa_bytes);
    const uint32_t lds_sb_wave = to_sgpr(lds0 + kMoeScaleBase + kMoeScaleA + (uint32_t)(w * 256));

    // A-side offsets do not depend on the work item: LDS row R of the A tile is row
    // row_start + R of the K-step's contiguous [S][128] block (rows past the tile's count are
    // other rows of the matrix, or out of range = zero, and their results are never stored).
    uint32_t voff_a[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) voff_a[i] = (uint32_t)(8 * (i * NW + w) + (lane >> 3)) * 128u + chunk16 * 16u;
    // scales of kMoeBM / 8 rows per wave: kMoeBM / 16 lanes x 16 bytes
    const uint32_t voff_sa = (uint32_t)(w * sa_bytes + lane * 16);
    constexpr uint64_t kSaMask = (1ull << (kMoeBM / 16)) - 1ull;

    // All loads of K-step kt of item `a` into `stage`. For an invalid item or past the end of K
    // they are issued against zero-sized buffers (no traffic), which keeps the number of
    // outstanding loads per K-step uniform.
    auto issue_tile = [&](const MoeAddr& a, int stage, int kt) {
        v4i sa = srd_a, sb = a.srd_b, ssa = srd_sa, ssb = a.srd_sb;
        if (!a.valid || kt >= nk) { sa.z = 0; sb.z = 0; ssa.z = 0; ssb.z = 0; }
        const uint32_t row_base = (uint32_t)kt * (uint32_t)p.S + (uint32_t)a.row_start;
        const uint32_t dst = lds_wave + (uint32_t)stage * kMoeStage;
        const uint32_t sadst = lds_sa_wave + (uint32_t)stage * kMoeScaleStage;
        const uint32_t sbdst = lds_sb_wave + (uint32_t)stage * kMoeScaleStage;
#pragma unroll
        for (int i = 0; i < NA; ++i) dma16(sa, dst + i * NW * 1024, voff_a[i], row_base * 128u);
        const bool last = (kt == nk - 1) && tail_oob;  // 16-byte chunks past the end of K read as zero
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dma16(sb, dst + kMoeATile + i * NW * 1024, last ? 0x80000000u : a.voff_b[i], (uint32_t)kt * 128u);
        dma16_lanes(ssa, sadst, voff_sa, row_base * 8u, kSaMask);
        dma4(ssb, sbdst, a.voff_sb, (uint32_t)kt * 8u);
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    // stage 0 addresses; a K-step on stage st adds st * kMoeStage (scales: st * kMoeScaleStage)
    const uint32_t a_lo0 = lds0 + wm * 2048 + rd_lo, a_hi0 = lds0 + wm * 2048 + rd_hi;
    const uint32_t b_lo0 = lds0 + kMoeATile + wn * (64 * 128) + rd_lo;
    const uint32_t b_hi0 = lds0 + kMoeATile + wn * (64 * 128) + rd_hi;
    const uint32_t sa_rd0 = lds0 + kMoeScaleBase + (wm * 16 + r) * 8u;
    const uint32_t sb_rd0 = lds0 + kMoeScaleBase + kMoeScaleA + (wn * 64 + r) * 8u;
    const uint32_t sh = 8u * g;  // byte g of each scale dword belongs to this lane
    struct Frag4 { v4i lo, hi; };
    auto rd_frag = [&](uint32_t lo, uint32_t hi, int imm) -> Frag4 {
        Frag4 f;
        f.lo = *(lds_v4i_t*)(uintptr_t)(lo + imm);
        f.hi = *(lds_v4i_t*)(uintptr_t)(hi + imm);
        return f;
    };
    auto rd_scale = [&](uint32_t base, int f) -> v2i {
        v2i s = *(lds_v2i_t*)(uintptr_t)(base + f * 128);
        s.x = (int)((uint32_t)s.x >> sh);
        s.y = (int)((uint32_t)s.y >> sh);
        return s;
    };

    v4f acc[MT][NT];
    MoeAddr cur, nxt;
    // Inline asm (not the builtin) so that the MFMAs keep their place relative to the loads that
    // are issued before / after them: a builtin call is free to sink below the asm statements.
    auto mfma = [&](v4f& c, const v4i& x, const v4i& y, int sx, int sy) {
        asm volatile(
            "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
            : "+v"(c)
            : "v"(x), "v"(y), "v"(sx), "v"(sy));
    };

    // MFMAs of one K-step on LDS stage st. Fragments past the tile's row count are skipped (the
    // condition is uniform for the wave).
    auto compute = [&](int st, int rows) {
        uint32_t a_lo = a_lo0 + (uint32_t)st * kMoeStage, a_hi = a_hi0 + (uint32_t)st * kMoeStage;
        uint32_t b_lo = b_lo0 + (uint32_t)st * kMoeStage, b_hi = b_hi0 + (uint32_t)st * kMoeStage;
        uint32_t sa_rd = sa_rd0 + (uint32_t)st * kMoeScaleStage, sb_rd = sb_rd0 + (uint32_t)st * kMoeScaleStage;
        // keep the (large) bases in registers so that fragment offsets stay immediates
        asm volatile("" : "+v"(a_lo), "+v"(a_hi), "+v"(b_lo), "+v"(b_hi), "+v"(sa_rd), "+v"(sb_rd));
        Frag4 bf[NT];
        v2i bs[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            bf[n] = rd_frag(b_lo, b_hi, n * 2048);
            bs[n] = rd_scale(sb_rd, n);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (16 * (2 * m + wm) < rows) {
                const Frag4 af = rd_frag(a_lo, a_hi, m * 4096);
                const v2i as = rd_scale(sa_rd, 2 * m);
#pragma unroll
                for (int n = 0; n < NT; ++n) mfma(acc[m][n], bf[n].lo, af.lo, bs[n].x, as.x);
#pragma unroll
                for (int n = 0; n < NT; ++n) mfma(acc[m][n], bf[n].hi, af.hi, bs[n].y, as.y);
            }
        }
    };

    auto epilogue = [&](const MoeAddr& a) {
        const int rows = a.rows, row_start = a.row_start, n0 = a.n0;
        if (MODE == 1) {
            uint16_t* out = (uint16_t*)p.out0;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * (2 * m + wm) + (int)r;
                if (row >= rows) continue;
                const size_t pos = (size_t)(row_start + row);
#pragma unroll
                for (int q = 0; q < NT / 2; ++q) {
                    const int col = n0 + wn * 64 + 32 * q + 8 * (int)g;
                    if (col + 8 > p.N) continue;  // N % 8 == 0
                    v4f x = acc[m][2 * q], y = acc[m][2 * q + 1];
                    if (EXT && p.bias) {
                        const float* bb = p.bias + (size_t)a.expert * p.N + col;
                        x += *(const v4f*)bb;
                        y += *(const v4f*)(bb + 4);
                    }
                    v4i o4;
                    o4.x = pack_bf16(x.x, x.y); o4.y = pack_bf16(x.z, x.w);
                    o4.z = pack_bf16(y.x, y.y); o4.w = pack_bf16(y.z, y.w);
                    *(v4i*)(out + pos * p.N + col) = o4;
                }
            }
        } else {
            // h goes out as K-step-major tiles for the down GEMM: column c of row pos lives in
            // K-step c / 256 at byte (c % 256) / 2; this wave's 32 columns are one MX block.
            uint8_t* hq = (uint8_t*)p.out0;
            const int hcol0 = n0 + 32 * wn;
            const bool col_ok = hcol0 < p.N;
            const size_t kt2 = (size_t)(hcol0 >> 8);
            const int byte0 = ((hcol0 & 255) >> 1) + 4 * (int)g, blk = (hcol0 & 255) >> 5;
            // extended epilogue: biases of this lane's 8 h columns hcol0 + 8 g .. +8
            float bg[8], bu[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) bg[i] = bu[i] = 0.f;
            if (EXT && p.bias && col_ok) {
                const float* bb = p.bias + (size_t)a.expert * 2 * p.N;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int c = hcol0 + 8 * (int)g + i;
                    bg[i] = bb[p.interleaved ? 2 * c : c];
                    bu[i] = bb[p.interleaved ? 2 * c + 1 : p.N + c];
                }
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * (2 * m + wm) + (int)r;
                if (16 * (2 * m + wm) >= rows) continue;  // uniform: the whole fragment is padding
                float h[8];
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const v4f gt = acc[m][2 * q], up = acc[m][2 * q + 1];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float gv = gt[j];
                        h[4 * q + j] = EXT ? glu_act(p.act, gv + bg[4 * q + j], up[j] + bu[4 * q + j], p.alpha, p.limit)
                                           : silu_mul(gv, up[j]);
                    }
                }
                float amax = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[i]));
                amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                const int e = mx_block_exponent(amax);
                if (row < rows && col_ok) {
                    const size_t tile_row = kt2 * p.S + (size_t)(row_start + row);
                    *(uint32_t*)(hq + tile_row * 128 + byte0) = pack8_e2m1(h, e);
                    if (g == 0) p.out_scales[tile_row * 8 + blk] = (uint8_t)(e + 127);
                }
            }
        }
    };

    // Stream of K-steps over this workgroup's items through a ring of three LDS stages: the
    // loads of the next two stream positions are in flight while one position is computed,
    // across item boundaries (one position ahead only when an item has a single K-step).
    const int depth = nk >= 2 ? 2 : 1;
    int st = 0;  // stage of the stream position being computed
    make_addr(it, cur);
    issue_tile(cur, 0, 0);
    if (depth == 2) issue_tile(cur, 1, 1);
    for (;;) {
        make_addr(it + it_stride, nxt);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
        for (int kt = 0; kt < nk; ++kt) {
            // this wave's part of the current position has landed (younger positions may fly)
            if (depth == 2) wait_vmcnt<kDma>(); else wait_vmcnt<0>();
            block_barrier();   // ... everyone's; and everyone is done with the previous position
            const int ahead = kt + depth;
            int stage_ahead = st + depth;
            if (stage_ahead >= 3) stage_ahead -= 3;
            // The texture-address unit needs about as long to take a K-step's loads as the
            // matrix pipes need for its MFMAs: the first wave of each SIMD issues its loads
            // before computing, the second one after, so that the two overlap.
            if (wm == 0) {
                if (ahead < nk) issue_tile(cur, stage_ahead, ahead);
                else issue_tile(nxt, stage_ahead, ahead - nk);
            }
            compute(st, cur.rows);
            if (wm == 1) {
                if (ahead < nk) issue_tile(cur, stage_ahead, ahead);
                else issue_tile(nxt, stage_ahead, ahead - nk);
            }
            st = st == 2 ? 0 : st + 1;
        }
        mfma_drain_vgpr(acc);
        epilogue(cur);
        it += it_stride;
        if (it >= it_end) break;
        cur = nxt;
    }
    wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup retires
}

// ------------------------------------------------------- grouped GEMM, pre-shuffled weights
// Weight-streaming grouped GEMM for the pre-shuffled layout. At MoE shapes the grouped GEMMs are
// bound by reading every expert's weights once from HBM, so the kernel is built around keeping
// as many weight bytes in flight per CU as possible and around reading them once:
//   * weights never touch LDS: the pre-shuffled layout stores, for every (expert, n-tile, K-step)
//     the MFMA B fragments as contiguous 1 KiB pieces (lane l's 16 bytes at 16*l), and each wave
//     loads its eight straight into registers three positions ahead of their use (a ring of four
//     register sets); their e8m0 scales come the same way;
//   * a work item covers up to 192 rows of an expert (12 activation fragments), so that an expert
//     with a few rows more than 128 still needs one pass over its weights;
//   * only the activation tile (shared by the waves, re-read from L2) goes through LDS, in four
//     stages filled by direct global->LDS loads. Loads return in order.
// One workgroup of 4 waves per CU, one wave per SIMD. Wave W owns weight rows [64 W, +64) of the
// 256-row tile (four fragments) x all rows of the item: 192 accumulator registers per lane,
// updated in place in AGPRs. The K-step stream runs across item boundaries. All vector-memory
// operations are inline asm and counted by hand (the compiler never waits for them). Results are
// bit-identical to moe_mxfp4_gemm_kernel (same accumulation order per output element).
//   * the 32 h columns of a wave are exactly one MX block, so the gate+up epilogue needs no
//     exchange between waves, no LDS and no workgroup barrier: block maxima and a row's 16 packed
//     bytes are gathered inside the wave by swapping rows of 16 lanes in registers
//     (v_permlane16_swap / v_permlane32_swap), one 16-byte store per 16 rows;
//   * the epilogue of row fragment M - 1 runs right behind the MFMAs of fragment M in the item's
//     last K-step, and the loads of the position three ahead are spread over the fragments of every
//     K-step, the last one included: the wave keeps requesting weights while it finishes an item.
// Per position a wave issues 17 loads: six 1 KiB pieces of the activation tile and its 384 bytes of
// row scales (global -> LDS, four stages), eight 1 KiB weight fragments and two scale dwords
// (global -> VGPRs, four register sets). Position q's loads are issued during position q - 3; they
// return in order, so at the start of position q everything of it has landed when at most the 34
// loads of positions q + 1 and q + 2 are outstanding.
// Measured at the GPT-OSS-like shape (kernel trace, us, gate+up / down): 275 / 148; without
// epilogues 227 / 115; loads, waits and barriers only 206 / 103; the K loop's MFMAs and LDS reads
// on empty loads 148 / 78. The K loop hides behind the weight stream, the epilogue does not. An
// epilogue copy per register set (four times the code) cost another 7 %: the loop then no longer
// fits the instruction cache. Requesting the weights of one or two further positions into L2 at
// the start of an item's last position changed nothing / cost 2 %; parking four fragments'
// accumulators in the spare AGPRs and finishing them in the next item's first position cost
// 6 us per layer: not kept. A predecessor with 8 waves (two per SIMD, 32 weight rows per wave,
// an LDS exchange in the gate+up epilogue) took 293 / 152 us with the plain epilogues and, for the
// extended ones, 9 us more per layer than this kernel; it is no longer in the tree.
//
// A8: the activations are MXFP8 (e4m3 elements, 256 bytes per row and K-step, same e8m0 scale
// layout) and the MFMA is the mixed form (fp4 weights x fp8 activations, 32 cycles). The
// activation tile is kept as two half-tiles of 128-byte rows (K halves), so that the LDS
// swizzle, the load pieces and the fragment addressing stay those of the FP4 tile; a lane's
// 32 bytes of a K half are the 16-byte chunks g and g + 4. Items have up to 128 rows then
// (four 33 KiB stages), and the gate+up epilogue re-quantizes h to MXFP8.
// EXT: biases / clamped SwiGLU / interleaved source rows in the epilogue.
// GATHER (gate+up, plain epilogue): the item's rows are fetched by token from x quantized once per
// token, and their scales once per 16 K-steps; see the kernel body. 16 loads per position then.
// NT: the weight fragments are loaded with the non-temporal hint. When an expert's rows fit one
// item its weights are read exactly once, and keeping them out of the caches leaves the L2 to the
// activations: at the GPT-OSS-like shape the layer takes 0.257 instead of 0.292 ms at 64 tokens,
// 0.322 instead of 0.355 at 1024, 0.448 instead of 0.467 at 4096. With several items per expert and
// n-tile (16384 tokens: 512 rows per expert) the later ones would fetch the weights from HBM again
// instead of from L2 (1.32 against 1.29 ms; 65536 tokens: 5.24 against 4.87): the host sets NT by
// the average number of rows per expert.
constexpr int kStBM = 192;                              // rows per work item
template <bool A8, bool GATHER>
struct S4Cfg {
    // rows per work item: what four LDS stages of the activation tile leave room for. MXFP8 rows are
    // twice as long: 144 rows (random routing of 4096 tokens gives 128 +- 11 rows per expert: with 128-row
    // items every second expert needed a second pass over its weights), 128 when the row scales' two
    // super-step buffers have to fit as well
    static constexpr int kBM = A8 ? (GATHER ? 128 : 144) : kStBM;
    static constexpr int kRow = A8 ? 256 : 128;        // activation bytes per row and K-step
    static constexpr int kATile = kBM * kRow;
    static constexpr int kStage = GATHER ? kATile : kATile + kBM * 8;    // + row scales of the position (not GATHER)
    static constexpr int kScaleTile = kBM * 128;       // GATHER: row scales of 16 K-steps, two buffers behind the stages
    static constexpr int kGroups = (kBM + 31) / 32;    // groups of 32 rows: wave w loads rows 8 w .. +8 of each
    static constexpr int kPieces = (A8 ? 2 : 1) * kGroups;   // 1 KiB activation loads per wave and position
    // a last group that is not full: its pieces of the waves past the tile's end go to a dump area
    static constexpr int kDump = kBM % 32 ? 4096 : 0;
    static constexpr int kLds = 4 * kStage + (GATHER ? 2 * kScaleTile : 0) + kDump;   // 102 / 144 KiB (MXFP8: 149 / 160)
};
static_assert(S4Cfg<true, true>::kLds <= 160 * 1024 && S4Cfg<false, true>::kLds <= 160 * 1024 &&
              S4Cfg<true, false>::kLds <= 160 * 1024 && S4Cfg<false, false>::kLds <= 160 * 1024, "LDS of a CU");
constexpr int kS4Ahead = 3;  // positions between fetch and compute (two measure the same)

template <int MODE, bool EXT, bool A8, bool GATHER = false, bool NT = false>
__global__ __launch_bounds__(256) void moe_mxfp4_stream4_kernel(const MoeGemmParams p) {
    static_assert(!GATHER || (MODE == 0 && !EXT), "rows are gathered by the gate+up kernel with the plain epilogue only");
    using Cfg = S4Cfg<A8, GATHER>;
    // GATHER (gate+up kernel, plain epilogue): the activation rows are fetched by token; the quantized x
    // is then stored once per token instead of once per routed slot (see tok_cur below), and its row
    // scales are stored 16 K-steps ("super-step") to a 128-byte row and fetched once per super-step
    // instead of once per position. (With the extended epilogue's registers on top, the slot
    // registers no longer fit.) Measured at the GPT-OSS-like shape, layer time with / without: 64 to
    // 4096 tokens 5-7 us less (the quantization rides in the sort's launch and writes a quarter of
    // the bytes), 16384 tokens 30 us more, 65536 tokens 70 us more: every XCD then reads all of x
    // instead of its experts' rows, and x no longer stays in its L2. The host picks by the size of x.
    constexpr int kBM = Cfg::kBM, kRow = Cfg::kRow, kATile = Cfg::kATile;
    constexpr int kStage = Cfg::kStage, kScaleTile = Cfg::kScaleTile;
    constexpr int kPieces = Cfg::kPieces, kGroups = Cfg::kGroups;
    constexpr int kScaleLoads = GATHER ? 0 : 1;
    constexpr int kLoads = kPieces + kScaleLoads + 10;   // + 8 weight fragments, 2 weight scale dwords
    constexpr int MT = kBM / 16;
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    const int lane = lane_id(), w = wave_id();
    const int n_items = scalar_load_x1(p.num_items);
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int it_stride = ((int)gridDim.x - xcd + kNumXcd - 1) / kNumXcd;  // workgroups on this XCD
    const int per_xcd = (n_items + kNumXcd - 1) / kNumXcd;
    const int it0 = xcd * per_xcd + slot;
    const int it_end = min(n_items, (xcd + 1) * per_xcd);
    if (it0 >= it_end) return;

    const int Kb = p.K >> 1;
    const int nk = (Kb + 127) >> 7;
    const int a_rows = GATHER ? p.a_rows : p.S;   // rows of the activation matrices
    const v4i srd_a = make_srd(p.A, (uint32_t)nk * (uint32_t)a_rows * (uint32_t)kRow);
    const v4i srd_sa = make_srd(p.SA, GATHER ? (uint32_t)((nk + 15) >> 4) * (uint32_t)a_rows * 128u
                                             : (uint32_t)nk * (uint32_t)a_rows * 8u);

    // ---- cursors over the stream of (item, K-step) positions of this workgroup ---------------
    struct Cursor { int it, kt, expert, row_start, rows, n_tile; bool valid; };
    auto load_item = [&](Cursor& c) __attribute__((always_inline)) {
        c.valid = c.it < it_end;
        const v4i item = scalar_load_x4(p.items + (c.valid ? c.it : it_end - 1));
        c.expert = item.x; c.row_start = item.y; c.rows = item.z; c.n_tile = item.w;
    };
    // An item takes nk4 positions, nk rounded up to a multiple of four (the length of the ring of
    // register sets): its last position is then always one of set 3, and the epilogue code exists
    // once instead of once per set. The padding positions fetch and compute nothing.
    const int nk4 = (nk + 3) & ~3;
    Cursor cc{it0, 0}, cf{it0, 0};  // compute, fetch (three positions ahead)
    load_item(cc);
    cf = cc;
    // per fetch item: weight and weight-scale descriptors, rows rounded up to fragments
    v4i cf_srd_b, cf_srd_sb;
    auto cf_descriptors = [&]() __attribute__((always_inline)) {
        cf_srd_b = make_srd(p.B + (size_t)cf.expert * p.b_expert_stride + (size_t)cf.n_tile * nk * kMoeBTile,
                            cf.valid ? (uint32_t)nk * kMoeBTile : 0u);
        cf_srd_sb = make_srd(p.SB + (size_t)cf.expert * p.sb_expert_stride + (size_t)cf.n_tile * nk * kMoeScaleB,
                             cf.valid ? (uint32_t)nk * kMoeScaleB : 0u);
    };
    cf_descriptors();
    // EXT: the lane's bias values. They are fetched when the FETCH cursor enters an item (four
    // 16-byte loads into bias_nxt: extra loads in the counted stream, which only makes the waits
    // stricter) and taken over when the compute cursor enters it, three positions later. (Fetching
    // them in the item's last K-step through the scalar cache stalled the wave for the latency of
    // two dependent loads per item: 62 us per layer at the GPT-OSS-like shape.)
    // MODE 0: lane (r, g) needs gate / up biases of h columns 128 n_tile + 32 w + 16 o + 4 g .. +4:
    // loads 2 o / 2 o + 1 = gate / up (plain row order) or the 8 interleaved floats (gate and up
    // alternating). MODE 1: output columns 256 n_tile + 64 w + 32 o + 8 g .. +8: loads 2 o, 2 o + 1.
    // Columns past N read other experts' values or zeros; their results are dropped.
    float bias_a[2][4], bias_b[2][4];  // MODE 0: [pair][j] gate / up; MODE 1: [pair][j] columns 8 g + j / 8 g + 4 + j
    v4f bias_nxt[4];
    // (range-checked: the lanes of an n-tile's columns past N index past their expert's values, for the
    // last expert past the array: they read zeros)
    const v4i srd_bias = make_srd(p.bias, EXT && p.bias ? p.bias_bytes : 0u);
    auto request_bias = [&]() __attribute__((always_inline)) {
        if constexpr (EXT) {
            const uint32_t gq = (uint32_t)(lane >> 4);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int o = q >> 1, part = q & 1;
                uint32_t idx;  // float index into the bias array
                if (MODE == 1) {
                    idx = (uint32_t)cf.expert * (uint32_t)p.N + (uint32_t)(cf.n_tile * 256 + 64 * w + 32 * o) + 8u * gq + 4u * part;
                } else {
                    const uint32_t hcol = (uint32_t)(cf.n_tile * 128 + 32 * w + 16 * o) + 4u * gq;
                    idx = (uint32_t)cf.expert * 2u * (uint32_t)p.N +
                          (p.interleaved ? 2u * hcol + 4u * part : (uint32_t)(part * p.N) + hcol);
                }
                v4f& dst = bias_nxt[q];
                const v4i rs = srd_bias;
                const uint32_t voff = idx * 4u;
                // (s_nop 4: the descriptor may have been restored from a spill slot by a vector-ALU
                // instruction directly in front of the statement)
                asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(dst) : "v"(voff), "s"(rs) : "memory");
            }
        }
    };
    auto adopt_bias = [&]() __attribute__((always_inline)) {
        if constexpr (EXT) {
#pragma unroll
            for (int o = 0; o < 2; ++o) {
                const v4f x0 = bias_nxt[2 * o], x1 = bias_nxt[2 * o + 1];
                if (MODE == 0 && p.interleaved) {
                    bias_a[o][0] = x0.x; bias_b[o][0] = x0.y; bias_a[o][1] = x0.z; bias_b[o][1] = x0.w;
                    bias_a[o][2] = x1.x; bias_b[o][2] = x1.y; bias_a[o][3] = x1.z; bias_b[o][3] = x1.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) { bias_a[o][j] = x0[j]; bias_b[o][j] = x1[j]; }
                }
            }
        }
    };
    // GATHER: byte offset of the lane's row inside a K-step plane of A for each activation piece i
    // (the row is 8 (4 i + w) + lane / 8), plus the lane's 16-byte chunk: for the fetch item
    // (tok_cur) and, as raw slot numbers still in flight, for the item after it (tok_nxt). The slots
    // of an item are requested one item ahead: by the time the fetch cursor reaches it, at least four
    // positions of counted loads have been waited for behind them. They are extra loads in the
    // counted stream; the waits only become stricter by them. Rows past the item (the rest of its
    // last fragment, or past the end of the list, which reads as slot 0) map to some valid token;
    // their results are dropped.
    // piece i of the activation (half-)tile = rows 8 (4 i + w) .. +8; the swizzle of a row depends
    // on its bits 1..3, i.e. on w and the lane only
    const uint32_t chunk16 = swz_chunk(8 * w + (lane >> 3), lane & 7);
    constexpr int kNp = kGroups;
    constexpr int kTok = GATHER ? kNp : 1;
    uint32_t tok_cur[kTok], tok_nxt[kTok];
    const v4i srd_slots = make_srd(p.row_slots, GATHER ? (uint32_t)p.S * 4u : 0u);
    auto request_tokens = [&](int row_start) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < kTok; ++q) {
            const uint32_t voff = (uint32_t)(row_start + 8 * (4 * q + w) + (lane >> 3)) * 4u;
            uint32_t& dst = tok_nxt[q];
            const v4i rs = srd_slots;
            // (once per item; s_nop 4: the descriptor may have been restored from a spill slot by a vector-ALU
            // instruction directly in front of the statement)
            asm volatile("s_nop 4\n\tbuffer_load_dword %0, %1, %2, 0 offen" : "=v"(dst) : "v"(voff), "s"(rs) : "memory");
        }
    };
    auto adopt_tokens = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < kTok; ++q) {
            const uint32_t slot = tok_nxt[q];
            const uint32_t tok = p.topk_magic ? __umulhi(slot, p.topk_magic) : slot;
            tok_cur[q] = tok * (uint32_t)kRow + chunk16 * 16u;
        }
    };
    // requests the slots of the item after the fetch item
    auto request_next_item = [&]() __attribute__((always_inline)) {
        const int it = min(cf.it + it_stride, it_end - 1);
        const v4i item = scalar_load_x4(p.items + it);
        request_tokens(item.y);
    };
    // GATHER: row scales. SA is [ceil(nk / 16)][a_rows][128]: a row's 8 scale bytes of K-step kt sit at
    // byte 8 (kt % 16) of its 128-byte row of super-step kt / 16. When the fetch cursor enters a
    // super-step, the wave fetches the scale rows of the rows it fetches activation pieces for into one
    // of two LDS buffers (the compute cursor is at most three positions behind, in this super-step or
    // the one before). A row's eight 16-byte chunks are stored rotated by bits 1..3 of the row number
    // (chunk c at position c ^ key), which spreads the 16 rows a fragment read touches over all banks.
    // Chunks past the super-step's last K-step are not fetched (their lanes write zeros).
    const uint32_t lds_ss = (uint32_t)(uintptr_t)smem + 4u * kStage;
    const uint32_t ss_key = (uint32_t)(4 * w + (lane >> 4)) & 7u;       // key of the rows this lane fetches
    const uint32_t ss_chunk = ((uint32_t)lane & 7u) ^ ss_key;           // the chunk it fetches
    uint32_t cf_ss = kScaleTile, cc_ss = kScaleTile;   // byte offset of the cursor's buffer (toggled on entering a super-step)
    auto fetch_scale_rows = [&]() __attribute__((always_inline)) {
        cf_ss ^= (uint32_t)kScaleTile;
        const int rows_up = cf.valid ? (cf.rows + 15) & ~15 : 0;
        const int chunks = (min(16, nk - cf.kt) + 1) >> 1;
        const uint32_t kill = (int)ss_chunk >= chunks ? 0x80000000u : 0u;
#pragma unroll
        for (int i = 0; i < kNp; ++i) {
            v4i ssa = srd_sa;
            if (8 * (4 * i + w) >= rows_up) ssa.z = 0;
            uint32_t base = tok_cur[i] - chunk16 * 16u;   // token * kRow
            if (A8) base >>= 1;
            dma16(ssa, to_sgpr(lds_ss + cf_ss + (uint32_t)(w * 1024 + i * 4096)), (base + ss_chunk * 16u) | kill,
                  (uint32_t)(cf.kt >> 4) * (uint32_t)a_rows * 128u);
        }
    };
    if constexpr (GATHER) {
        request_tokens(cf.row_start);
        wait_vmcnt<0>();
        adopt_tokens();
        request_next_item();
        fetch_scale_rows();
    }
    if constexpr (EXT) {
        request_bias();
        wait_vmcnt<0>();
        adopt_bias();
    }
    // The 2 kNp loads a change of the fetch item adds (slots, scale rows) sit between the counted loads
    // of two positions: the waits of the next three positions allow for them.
    int cf_extra = 0;
    auto advance_cf = [&]() __attribute__((always_inline)) {
        if (++cf.kt == nk4) {
            cf.kt = 0; cf.it += it_stride; load_item(cf); cf_descriptors();
            // the counter of outstanding vector-memory operations has six bits: room for the four bias loads
            if constexpr (EXT && kS4Ahead * kLoads + 4 > 63) wait_vmcnt<63 - 4>();
            request_bias();
            if constexpr (GATHER) { adopt_tokens(); request_next_item(); cf_extra = 3; }
        }
        if constexpr (GATHER)
            if ((cf.kt & 15) == 0) fetch_scale_rows();
    };

    // ---- loads of one position ------------------------------------------------------------------
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kATile + (uint32_t)w * (2u * kBM));
    const uint32_t voff_a0 = (uint32_t)(8 * w + (lane >> 3)) * (uint32_t)kRow + chunk16 * 16u;  // + 32 i rows (+ 128 for the second K half)
    const uint32_t voff_sa = (uint32_t)(w * 2 * kBM + lane * 16);   // the row scales of rows [kBM / 4 * w, + kBM / 4)
    const uint32_t voff_b = lane * 16, voff_sb = lane * 4;
    v4i bw[4][8];   // [position mod 4][4 * (weight fragment pair) + 2 * fragment + K half]
    int bsc[4][2];  // [position mod 4][pair]: the lane's scale bytes, byte 2 * half + fragment
    // Bytes of the last K-step that lie inside K (the layout pads every row to whole K-steps with
    // zeros): lane l's 16 bytes of half h start at byte 64 h + 16 (l / 16) of the K-step. Lanes
    // past the end get bit 31 in their offset: outside the buffer, so the load returns the same
    // zeros without fetching them.
    const int last_valid = Kb - (nk - 1) * 128;
    // load L (0 .. kLoads - 1) of the fetch position, into LDS stage / register set P
    auto fetch_load = [&]<int P, int L>() __attribute__((always_inline)) {
        if constexpr (L < kPieces) {
            constexpr int i = L % kGroups, khalf = L / kGroups;
            const int rows_up = cf.valid && cf.kt < nk ? (cf.rows + 15) & ~15 : 0;
            v4i sa = srd_a;
            if (8 * (4 * i + w) >= rows_up) sa.z = 0;  // past the item's last fragment: nothing is fetched
            uint32_t dst = lds_wave + (uint32_t)(P * kStage + khalf * (kBM * 128) + i * 4096);
            // a piece past the tile's end (last, partial group of 32 rows): never holds rows, lands in the dump area
            if constexpr (32 * i + 32 > kBM)
                if (8 * (4 * i + w) >= kBM) dst = lds_wave + (uint32_t)(Cfg::kLds - Cfg::kDump);
            if constexpr (GATHER) {
                dma16(sa, dst, tok_cur[i],
                      (uint32_t)cf.kt * (uint32_t)a_rows * (uint32_t)kRow + (uint32_t)(khalf * 128));
            } else {
                const uint32_t row_base = (uint32_t)cf.kt * (uint32_t)p.S + (uint32_t)cf.row_start;
                dma16(sa, dst, voff_a0 + (uint32_t)(i * 32 * kRow + khalf * 128), row_base * (uint32_t)kRow);
            }
        } else if constexpr (L < kPieces + kScaleLoads) {
            v4i ssa = srd_sa;
            if (!cf.valid || cf.kt >= nk) ssa.z = 0;
            const uint32_t row_base = (uint32_t)cf.kt * (uint32_t)p.S + (uint32_t)cf.row_start;
            dma16_lanes(ssa, lds_sa_wave + (uint32_t)(P * kStage), voff_sa, row_base * 8u, (1ull << (kBM / 8)) - 1ull);
        } else if constexpr (L < kPieces + kScaleLoads + 8) {
            constexpr int f = L - kPieces - kScaleLoads, pair = f >> 2, half = f & 1;
            const int thr = cf.kt == nk - 1 ? 16 * min(max(last_valid - 64 * half, 0), 64) - 1 : 0x7fffffff;
            const uint32_t voff = voff_b | ((uint32_t)(thr - (int)voff_b) & 0x80000000u);
            const uint32_t soff = (uint32_t)cf.kt * kMoeBTile + (uint32_t)(2 * w + pair) * 4096u;
            v4i rs = cf_srd_b;
            if (cf.kt >= nk) rs.z = 0;
            // (the first weight load of a position starts with s_nop 4: the descriptor's size word may have
            // been restored from a spill slot by a vector-ALU instruction directly in front of the statement)
#define HK_WLOAD(PRE, POST)                                                                      \
    asm volatile(PRE "buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" POST                   \
                 : "=v"(bw[P][f])                                                                \
                 : "v"(voff), "s"(rs), "s"(soff), "n"(((f >> 1) & 1) * 2048 + half * 1024)       \
                 : "memory")
            if constexpr (f == 0) {
                if constexpr (NT) HK_WLOAD("s_nop 4\n\t", " nt"); else HK_WLOAD("s_nop 4\n\t", "");
            } else {
                if constexpr (NT) HK_WLOAD("", " nt"); else HK_WLOAD("", "");
            }
#undef HK_WLOAD
        } else if constexpr (L < kLoads) {
            constexpr int pair = L - kPieces - kScaleLoads - 8;
            int& dst = bsc[P][pair];
            v4i rss = cf_srd_sb;
            if (cf.kt >= nk) rss.z = 0;
            const uint32_t voff = voff_sb;
            asm volatile("buffer_load_dword %0, %1, %2, %3 offen"
                         : "=v"(dst)
                         : "v"(voff), "s"(rss), "s"((uint32_t)cf.kt * kMoeScaleB + (uint32_t)(2 * w + pair) * 256u)
                         : "memory");
        }
    };
    auto fetch_all = [&]<int P>() __attribute__((always_inline)) {
        [&]<int... L>(std::integer_sequence<int, L...>) __attribute__((always_inline)) {
            (fetch_load.template operator()<P, L>(), ...);
        }(std::make_integer_sequence<int, kLoads>{});
        advance_cf();
    };

    // ---- LDS -> registers (activation fragments) ------------------------------------------------
    const uint32_t r = lane & 15, g = lane >> 4;
    // MXFP4: the lane's 16 bytes of K half h are chunk g + 4 h of the row. MXFP8: its 32 bytes are
    // chunks g and g + 4 of the row of half-tile h. (An 8-register operand of this MFMA holds, in
    // lane group g, positions [16 g, +16) and [64 + 16 g, +16) of the 128 it contracts over, a
    // 4-register one positions [32 g, +32); the scale of positions [32 b, +32) comes from lane
    // group b for either operand. Measured with one-hot operands, not documented.)
    const uint32_t rd_half[2][2] = {
        {lds0 + r * 128u + swz_chunk(r, g) * 16u, lds0 + r * 128u + swz_chunk(r, g + 4) * 16u},
        {lds0 + (A8 ? kBM * 128u + r * 128u + swz_chunk(r, g) * 16u : r * 128u + swz_chunk(r, g + 4) * 16u),
         lds0 + kBM * 128u + r * 128u + swz_chunk(r, g + 4) * 16u}};
    const uint32_t sa_rd0 = lds0 + kATile + r * 8u;
    const uint32_t sh = 8u * g;  // byte g of each scale dword belongs to this lane

    v4f acc[MT][4];  // [row fragment][2 * pair + fragment]
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < 4; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
    auto mfma = [&](v4f& c, const v4i& x, const v4i& y, int sx, int sy) __attribute__((always_inline)) {
        asm volatile(
            "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
            : "+a"(c)
            : "v"(x), "v"(y), "v"(sx), "v"(sy));
    };
    // fp4 weights (4 registers) x fp8 activations (8 registers)
    auto mfma8 = [&](v4f& c, const v4i& x, const v8i& y, int sx, int sy) __attribute__((always_inline)) {
        asm volatile(
            "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4"
            : "+a"(c)
            : "v"(x), "v"(y), "v"(sx), "v"(sy));
    };

    // ---- epilogue of row fragment m of the compute item (its accumulators are final) -------------
    // Stores go through buffer descriptors that end at the item's last row: rows of the last
    // fragment beyond it (they belong to the next expert) are dropped by the range check, so the
    // epilogue needs no per-lane row test and no 64-bit address arithmetic. Lanes that do not
    // store at all carry bit 31 in their offset. Set up once per item by begin_epilogue().
    v4i st_srd0, st_srd1;     // MODE 0: packed h / its scales; MODE 1: the bf16 output
    uint32_t st_voff0 = 0, st_voff1 = 0;
    bool st_ok[2] = {false, false};  // MODE 0: [0] the wave's MX block lies inside N; MODE 1: its two 32-column groups
    auto begin_epilogue = [&]() __attribute__((always_inline)) {
        if (MODE == 1) {
            const uint32_t pitch = (uint32_t)p.N * 2u;
            st_srd0 = make_srd((uint8_t*)p.out0 + (size_t)cc.row_start * pitch, (uint32_t)cc.rows * pitch);
            const int wcol0 = cc.n_tile * 256 + 64 * w;  // N % 32 == 0: a group of 32 columns is valid as a whole
            st_ok[0] = wcol0 < p.N; st_ok[1] = wcol0 + 32 < p.N;
            st_voff0 = r * pitch + (uint32_t)(wcol0 + 8 * (int)g) * 2u;
        } else {
            const size_t row0 = (size_t)(cc.n_tile >> 1) * p.S + (size_t)cc.row_start;
            st_srd0 = make_srd((uint8_t*)p.out0 + row0 * kRow, (uint32_t)cc.rows * (uint32_t)kRow);
            st_srd1 = make_srd(p.out_scales + row0 * 8, (uint32_t)cc.rows * 8u);
            const uint32_t seg = (uint32_t)(cc.n_tile & 1) * (kRow / 2);  // the n-tile's 128 columns are half of a K-step row
            st_ok[0] = cc.n_tile * 128 + 32 * w < p.N;
            // MXFP4: the row's 16 bytes leave from its lane g = 0; MXFP8: its 32 bytes from lanes g = 0, 1
            if (A8) st_voff0 = g < 2 ? r * 256u + seg + 32u * (uint32_t)w + 16u * g : 0x80000000u;
            else st_voff0 = g == 0 ? r * 128u + seg + 16u * (uint32_t)w : 0x80000000u;
            st_voff1 = g == 0 ? r * 8u + 4u * (uint32_t)(cc.n_tile & 1) + (uint32_t)w : 0x80000000u;
        }
    };
    auto epilogue = [&]<int M>(bool drain) __attribute__((always_inline)) {
        // The accumulators are operands of this statement: the compiler sees no hazard behind the
        // MFMA statements and would otherwise move the reads of the accumulators up to them.
        asm volatile("" : "+a"(acc[M][0]), "+a"(acc[M][1]), "+a"(acc[M][2]), "+a"(acc[M][3]));
        // fragment M's MFMAs are followed by those of fragment M + 1 unless it was the item's last
        if (drain) asm volatile("s_nop 15\n\ts_nop 7" : "+a"(acc[M][0]), "+a"(acc[M][1]), "+a"(acc[M][2]), "+a"(acc[M][3]));
        if (MODE == 1) {
            // lane (r, g) holds, for row 16 M + r, the columns 64 w + 32 o + 8 g .. +8 (o = 0, 1)
#pragma unroll
            for (int o = 0; o < 2; ++o) {
                v4f x = acc[M][2 * o], y = acc[M][2 * o + 1];
                if (EXT)
#pragma unroll
                    for (int j = 0; j < 4; ++j) { x[j] += bias_a[o][j]; y[j] += bias_b[o][j]; }
                v4i o4;
                o4.x = pack_bf16(x.x, x.y); o4.y = pack_bf16(x.z, x.w);
                o4.z = pack_bf16(y.x, y.y); o4.w = pack_bf16(y.z, y.w);
                if (st_ok[o])
                    asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen offset:%3\n\ts_nop 1"
                                 :: "v"(o4), "v"(st_voff0), "s"(st_srd0), "n"(o * 64) : "memory");
            }
            st_voff0 += 32u * (uint32_t)p.N;  // 16 rows
        } else {
            // h = act(gate, up): lane (r, g) holds, for row 16 M + r, the h columns
            // 128 n_tile + 32 w + 16 o + 4 g .. +4 (o = 0, 1): the wave's 32 columns are one MX block
            float h[2][4];
            float amax = 0.f;
#pragma unroll
            for (int o = 0; o < 2; ++o) {
                const v4f gt = acc[M][2 * o], up = acc[M][2 * o + 1];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (EXT) h[o][j] = glu_act(p.act, gt[j] + bias_a[o][j], up[j] + bias_b[o][j], p.alpha, p.limit);
                    else h[o][j] = silu_mul(gt[j], up[j]);
                    amax = fmaxf(amax, fabsf(h[o][j]));
                }
            }
            // maximum over the four lanes (r, 0..3) of a row: rows of 16 lanes swapped in registers
            {
                const uint32_t a = __float_as_uint(amax);
                const auto s16 = __builtin_amdgcn_permlane16_swap(a, a, false, false);
                const uint32_t m1 = __float_as_uint(fmaxf(__uint_as_float(s16[0]), __uint_as_float(s16[1])));
                const auto s32 = __builtin_amdgcn_permlane32_swap(m1, m1, false, false);
                amax = fmaxf(__uint_as_float(s32[0]), __uint_as_float(s32[1]));
            }
            int e = A8 ? mx8_block_exponent(amax) : mx_block_exponent(amax);
            v4i o4;
            if (A8) {
                const float hv[8] = {h[0][0], h[0][1], h[0][2], h[0][3], h[1][0], h[1][1], h[1][2], h[1][3]};
                v2i pk = pack8_e4m3(hv, e);  // .x: columns 4 g .. +4 of the block's first 16, .y: of its second 16
                if (!st_ok[0]) { pk = v2i{0, 0}; e = 0; }  // columns past N (uniform): zeros with a scale of one
                // rows of 16 lanes swapped between the two registers: lane (r, 0) ends up with the
                // first 16 columns' codes of all four lanes, lane (r, 1) with the second 16's
                const auto q16 = __builtin_amdgcn_permlane16_swap((uint32_t)pk.x, (uint32_t)pk.y, false, false);  // [a0 b0 a2 b2], [a1 b1 a3 b3]
                const auto q02 = __builtin_amdgcn_permlane32_swap(q16[0], q16[0], false, false);  // [a0 b0 ..], [a2 b2 ..]
                const auto q13 = __builtin_amdgcn_permlane32_swap(q16[1], q16[1], false, false);  // [a1 b1 ..], [a3 b3 ..]
                o4 = v4i{(int)q02[0], (int)q13[0], (int)q02[1], (int)q13[1]};
            } else {
                const float scale = __uint_as_float(e > -127 ? (uint32_t)(e + 127) << 23 : 0x00400000u);
                uint32_t pk = 0;  // low half: columns 4 g .. +4 of the block's first 16, high half: of its second 16
                pk = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(pk, h[0][0], h[0][1], scale, 0);
                pk = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(pk, h[0][2], h[0][3], scale, 1);
                pk = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(pk, h[1][0], h[1][1], scale, 2);
                pk = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(pk, h[1][2], h[1][3], scale, 3);
                if (!st_ok[0]) { pk = 0; e = 0; }  // columns past N (uniform): zeros with a scale of one
                // every lane of a row gets the packed values of all four: p[g'] = pk of lane (r, g')
                const auto q16 = __builtin_amdgcn_permlane16_swap(pk, pk, false, false);       // [p0 p0 p2 p2], [p1 p1 p3 p3]
                const auto q02 = __builtin_amdgcn_permlane32_swap(q16[0], q16[0], false, false);  // p0, p2
                const auto q13 = __builtin_amdgcn_permlane32_swap(q16[1], q16[1], false, false);  // p1, p3
                // the row's 16 bytes: the first 16 columns' codes (low halves), then the second 16's
                o4.x = (int)__builtin_amdgcn_perm(q13[0], q02[0], 0x05040100u);
                o4.y = (int)__builtin_amdgcn_perm(q13[1], q02[1], 0x05040100u);
                o4.z = (int)__builtin_amdgcn_perm(q13[0], q02[0], 0x07060302u);
                o4.w = (int)__builtin_amdgcn_perm(q13[1], q02[1], 0x07060302u);
            }
            asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen\n\ts_nop 1"
                         :: "v"(o4), "v"(st_voff0), "s"(st_srd0) : "memory");
            asm volatile("buffer_store_byte %0, %1, %2, 0 offen"
                         :: "v"(e + 127), "v"(st_voff1), "s"(st_srd1) : "memory");
            st_voff0 += 16u * (uint32_t)kRow;
            st_voff1 += 16u * 8u;
        }
#pragma unroll
        for (int n = 0; n < 4; ++n) acc[M][n] = v4f{0.f, 0.f, 0.f, 0.f};
    };

    // ---- prologue: positions 0..2 -----------------------------------------------------------------
    fetch_all.template operator()<0>();
    fetch_all.template operator()<1>();
    fetch_all.template operator()<2>();

    // One stream position on LDS stage / register set P; the loads of the position three ahead go
    // to stage / set (P + 3) % 4, which the previous position has just finished with.
    auto step = [&]<int P>() __attribute__((always_inline)) {
        constexpr int PF = (P + kS4Ahead) % 4;
        if (GATHER && cf_extra > 0) {
            --cf_extra;
            wait_vmcnt<(kS4Ahead - 1) * kLoads + 2 * kNp>();
        } else {
            wait_vmcnt<(kS4Ahead - 1) * kLoads>();
        }
        block_barrier();  // everyone's part of this position's tile has landed; stage PF is free
#pragma unroll
        for (int f = 0; f < 8; ++f) asm volatile("" : "+v"(bw[P][f]));
        asm volatile("" : "+v"(bsc[P][0]), "+v"(bsc[P][1]));
        const int rows = cc.valid && cc.kt < nk ? cc.rows : 0;  // padding, or past the end of the stream: no MFMAs
        const int mt = (rows + 15) >> 4;
        const int mt_item = cc.valid ? (cc.rows + 15) >> 4 : 0;
        const bool last = P == 3 && cc.valid && cc.kt == nk4 - 1;
        if (last) {
            begin_epilogue();
        }
        int bs[8];  // scale of weight fragment f = 4 pair + 2 n + half: byte 2 half + n of the pair's dword
#pragma unroll
        for (int f = 0; f < 8; ++f) bs[f] = (int)((uint32_t)bsc[P][f >> 2] >> (8 * (2 * (f & 1) + ((f >> 1) & 1))));
        uint32_t a_rd[2][2];
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
            for (int j = 0; j < 2; ++j) a_rd[hh][j] = rd_half[hh][j] + (uint32_t)(P * kStage);
        uint32_t sa_rd = sa_rd0 + (uint32_t)(P * kStage);
        if constexpr (GATHER) {
            // the row's 8 bytes of this K-step in the scale buffer of the compute cursor's super-step
            if ((cc.kt & 15) == 0) cc_ss ^= (uint32_t)kScaleTile;
            sa_rd = lds_ss + cc_ss + r * 128u + (((((uint32_t)cc.kt & 15u) >> 1) ^ ((r >> 1) & 7u)) << 4) +
                    ((uint32_t)cc.kt & 1u) * 8u;
        }
        // bases in registers, offsets as immediates
        asm volatile("" : "+v"(a_rd[0][0]), "+v"(a_rd[1][0]), "+v"(sa_rd));
        if (A8) asm volatile("" : "+v"(a_rd[0][1]), "+v"(a_rd[1][1]));
        v4i af[3][2];
        v8i af8[3][2];
        v2i as[3];
        auto rd = [&](int m) __attribute__((always_inline)) {
            if constexpr (A8) {
                af8[m % 3][0] = lds_frag(a_rd[0][0], a_rd[0][1], m * 2048);
                af8[m % 3][1] = lds_frag(a_rd[1][0], a_rd[1][1], m * 2048);
            } else {
                af[m % 3][0] = *(lds_v4i_t*)(uintptr_t)(a_rd[0][0] + m * 2048);
                af[m % 3][1] = *(lds_v4i_t*)(uintptr_t)(a_rd[1][0] + m * 2048);
            }
            as[m % 3] = *(lds_v2i_t*)(uintptr_t)(sa_rd + m * (GATHER ? 2048 : 128));
        };
        if (mt > 0) { rd(0); rd(1); }
        auto frag = [&]<int M>() __attribute__((always_inline)) {
            if (M < mt) {
                if (M + 2 < MT) rd(M + 2);  // rows past the tile's count are readable, never used
                const int sa[2] = {(int)((uint32_t)as[M % 3].x >> sh), (int)((uint32_t)as[M % 3].y >> sh)};
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int n = 0; n < 4; ++n) {
                        const int f = 4 * (n >> 1) + 2 * (n & 1) + half;
                        if constexpr (A8) mfma8(acc[M][n], bw[P][f], af8[M % 3][half], bs[f], sa[half]);
                        else mfma(acc[M][n], bw[P][f], af[M % 3][half], bs[f], sa[half]);
                    }
            }
            // the position's loads, spread over the fragments
            fetch_load.template operator()<PF, M>();
            if constexpr (M + MT < kLoads) fetch_load.template operator()<PF, M + MT>();
            if constexpr (M + 2 * MT < kLoads) fetch_load.template operator()<PF, M + 2 * MT>();
            if constexpr (M >= 1) {
                if constexpr (P == 3)
                    if (last && M - 1 < mt_item) epilogue.template operator()<M - 1>(M >= mt);
            }
        };
        [&]<int... M>(std::integer_sequence<int, M...>) __attribute__((always_inline)) {
            (frag.template operator()<M>(), ...);
        }(std::make_integer_sequence<int, MT>{});
        advance_cf();
        if constexpr (P == 3)
            if (last && MT - 1 < mt_item) epilogue.template operator()<MT - 1>(true);
        if (++cc.kt == nk4) {
            // the fetch cursor entered this item three positions ago and is still in it (nk4 >= 4)
            cc = cf; cc.kt = 0;
            adopt_bias();
        }
    };
    // Four positions per trip (stages and register sets rotate); positions past the end of the
    // stream degenerate to their barrier and empty loads.
    while (cc.valid) {
        step.template operator()<0>();
        step.template operator()<1>();
        step.template operator()<2>();
        step.template operator()<3>();
    }
    wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup retires
}

// ------------------------------------------------------------------------------ un-permute
// y[t, :] = bf16( add[t, :] + sum_j w[t, j] * o[slot_to_pos[t*k + j], :] ), fp32 accumulation in
// choice order starting from add (bf16 [T, H], e.g. a shared expert's output) or from 0 when add
// is null.
// KU > 0: k <= KU, the token's positions and weights are read once and the k rows' loads of a column
// chunk are issued together; KU == 0: any k, one row at a time. Same operations in the same order.
// The rows of o are read exactly once: non-temporal loads (213 -> 187 us at T = 8192, k = 8,
// H = 7168, i.e. 5.7 TB/s; the GPT-OSS-like layer 10 us less).
// o has T * k rows; a position outside [0, T * k) (a caller's broken slot_to_pos) is not read and adds
// nothing, like an expert id out of range in the sort.
template <int KU>
__global__ __launch_bounds__(256) void moe_unpermute_kernel(const uint16_t* __restrict__ o,
                                                            const float* __restrict__ w,
                                                            const int32_t* __restrict__ slot_to_pos, int T,
                                                            int k, int H, const uint16_t* __restrict__ add,
                                                            uint16_t* __restrict__ y) {
    const int t = blockIdx.x;
    int pos[KU > 0 ? KU : 1];
    float wt[KU > 0 ? KU : 1];
#pragma unroll
    for (int j = 0; j < KU; ++j) {
        pos[j] = j < k ? slot_to_pos[(size_t)t * k + j] : -1;
        wt[j] = j < k ? w[(size_t)t * k + j] : 0.f;
    }
    const uint32_t n_rows = (uint32_t)T * (uint32_t)k;
    for (int c = threadIdx.x; c < H / 8; c += 256) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        v4i rows[KU > 0 ? KU : 1];
#pragma unroll
        for (int j = 0; j < KU; ++j)
            if ((uint32_t)pos[j] < n_rows) rows[j] = __builtin_nontemporal_load((const v4i*)(o + (size_t)pos[j] * H + c * 8));
        if (add) {
            const v4i raw = *(const v4i*)(add + (size_t)t * H + c * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] = __uint_as_float((uint32_t)raw[i] << 16);
                acc[2 * i + 1] = __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
            }
        }
        if constexpr (KU > 0) {
#pragma unroll
            for (int j = 0; j < KU; ++j)
                if ((uint32_t)pos[j] < n_rows) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[2 * i] += wt[j] * __uint_as_float((uint32_t)rows[j][i] << 16);
                        acc[2 * i + 1] += wt[j] * __uint_as_float((uint32_t)rows[j][i] & 0xffff0000u);
                    }
                }
        } else {
            for (int j = 0; j < k; ++j) {
                const int pj = slot_to_pos[(size_t)t * k + j];
                if ((uint32_t)pj >= n_rows) continue;
                const float wj = w[(size_t)t * k + j];
                const v4i raw = *(const v4i*)(o + (size_t)pj * H + c * 8);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] += wj * __uint_as_float((uint32_t)raw[i] << 16);
                    acc[2 * i + 1] += wj * __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
                }
            }
        }
        v4i out;
        out.x = pack_bf16(acc[0], acc[1]); out.y = pack_bf16(acc[2], acc[3]);
        out.z = pack_bf16(acc[4], acc[5]); out.w = pack_bf16(acc[6], acc[7]);
        *(v4i*)(y + (size_t)t * H + c * 8) = out;
    }
}

int moe_num_compute_units() {
    static std::atomic<int> cached[64];   // per device ordinal; 0 = not queried yet
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev >= 0 && dev < 64 && (cus = cached[dev].load(std::memory_order_relaxed)) > 0) return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 256;
    if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

void moe_launch_build_items(const int32_t* expert_offsets, int E, int bm, int n_tiles_n1, MoeItem* items1,
                            int n_tiles_n2, MoeItem* items2, int32_t* num_items, hipStream_t s) {
    MoeBuildItems b;
    b.bm = bm;
    b.items[0] = items1; b.items[1] = items2;
    b.n_tiles[0] = n_tiles_n1; b.n_tiles[1] = n_tiles_n2;
    // eight workgroups per list share the n-tiles (a thread otherwise writes ~100 items one by one)
    hipLaunchKernelGGL(moe_build_items_kernel, dim3(2, 8), dim3(512), 0, s, expert_offsets, E, b, num_items);
}

template <int MODE, bool EXT, bool A8, bool GATHER, bool NT>
static int launch_moe_stream_nt(MoeGemmParams p, int max_items, hipStream_t s) {
    constexpr int lds = S4Cfg<A8, GATHER>::kLds, threads = 256;
    const void* kern = (const void*)moe_mxfp4_stream4_kernel<MODE, EXT, A8, GATHER, NT>;
    static DeviceOnce configured;
    if (!set_lds_limit_once(kern, lds, configured)) return HK_ERR_LAUNCH;
    // persistent: one workgroup per CU, each walking its share of the item list
    const int grid = min(max_items, moe_num_compute_units());
    void* args[] = {&p};
    if (hipLaunchKernel(kern, dim3(grid), dim3(threads), args, lds, s) != hipSuccess) return HK_ERR_LAUNCH;
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}
// nt: non-temporal weight loads (see the kernel)
template <int MODE, bool EXT, bool A8, bool GATHER = false>
static int launch_moe_stream(MoeGemmParams p, int max_items, hipStream_t s, bool nt) {
    return nt ? launch_moe_stream_nt<MODE, EXT, A8, GATHER, true>(p, max_items, s)
              : launch_moe_stream_nt<MODE, EXT, A8, GATHER, false>(p, max_items, s);
}

template <int MODE, bool EXT>
static int launch_moe_gemm(MoeGemmParams p, int max_items, hipStream_t s) {
    auto kern = moe_mxfp4_gemm_kernel<MODE, EXT>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kMoeLds, configured)) return HK_ERR_LAUNCH;
    // persistent: one workgroup per CU, each walking its share of the item list
    const int grid = min(max_items, moe_num_compute_units());
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kMoeLds, s, p);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

}  // namespace hk

using namespace hk;

extern "C" int hk_mxfp4_quantize_rows(const void* x_bf16, int rows, int cols, void* packed, void* scales,
                                      int scale_pitch, void* stream) {
    if (!x_bf16 || !packed || !scales) return HK_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || (cols % 32) != 0 || scale_pitch < cols / 32 || (scale_pitch % 8) != 0)
        return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)x_bf16 | (uintptr_t)packed) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const long long threads = (long long)rows * scale_pitch * 4;
    hipLaunchKernelGGL(mx_quantize_rows_kernel<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t*)x_bf16, rows, cols, (uint8_t*)packed,
                       (uint8_t*)scales, scale_pitch);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_mxfp8_quantize_rows(const void* x_bf16, int rows, int cols, void* codes, void* scales,
                                      int scale_pitch, void* stream) {
    if (!x_bf16 || !codes || !scales) return HK_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || (cols % 32) != 0 || scale_pitch < cols / 32 || (scale_pitch % 8) != 0)
        return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)x_bf16 | (uintptr_t)codes) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const long long threads = (long long)rows * scale_pitch * 4;
    hipLaunchKernelGGL(mx_quantize_rows_kernel<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t*)x_bf16, rows, cols, (uint8_t*)codes,
                       (uint8_t*)scales, scale_pitch);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_unpermute_add(const void* o_bf16, const float* w, const int32_t* slot_to_pos, int T,
                                    int k, int H, const void* add_bf16_or_null, void* y_bf16, void* stream) {
    if (!o_bf16 || !w || !slot_to_pos || !y_bf16) return HK_ERR_NULL_POINTER;
    if (T <= 0 || k <= 0 || H <= 0 || (H % 8) != 0) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)o_bf16 | (uintptr_t)y_bf16 | (uintptr_t)add_bf16_or_null) & 15u) return HK_ERR_BAD_ALIGNMENT;
    auto kern = k <= 4 ? moe_unpermute_kernel<4> : k <= 8 ? moe_unpermute_kernel<8> : moe_unpermute_kernel<0>;
    hipLaunchKernelGGL(kern, dim3(T), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)o_bf16,
                       w, slot_to_pos, T, k, H, (const uint16_t*)add_bf16_or_null, (uint16_t*)y_bf16);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_unpermute(const void* o_bf16, const float* w, const int32_t* slot_to_pos, int T, int k,
                                int H, void* y_bf16, void* stream) {
    return hk_moe_unpermute_add(o_bf16, w, slot_to_pos, T, k, H, nullptr, y_bf16, stream);
}

extern "C" int hk_moe_mxfp4_preshuffle_bytes(int E, int N, int K, int mode, size_t* w_bytes, size_t* s_bytes) {
    if (!w_bytes || !s_bytes) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 32) != 0 || mode < 0 || mode > 2) return HK_ERR_BAD_SHAPE;
    const size_t n_tiles = mode != 1 ? ((size_t)N + 127) / 128 : ((size_t)N + 255) / 256;
    const size_t nk = ((size_t)K / 2 + 127) / 128;
    if ((double)E * (double)n_tiles * (double)nk * kMoeBTile >= 4e18) return HK_ERR_BAD_SHAPE;   // beyond size_t
    *w_bytes = (size_t)E * n_tiles * nk * kMoeBTile;
    *s_bytes = (size_t)E * n_tiles * nk * kMoeScaleB;
    return HK_OK;
}

extern "C" int hk_moe_mxfp4_preshuffle(const void* w, const void* scales, int scale_pitch, int E, int N, int K,
                                       int mode, void* out_w, void* out_s, void* stream) {
    if (!w || !scales || !out_w || !out_s) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 32) != 0 || scale_pitch < K / 32 || mode < 0 || mode > 2)
        return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)w | (uintptr_t)out_w) & 15u) return HK_ERR_BAD_ALIGNMENT;
    if (N > (1 << 30)) return HK_ERR_BAD_SHAPE;
    const int n_tiles = mode != 1 ? (N + 127) / 128 : (N + 255) / 256;
    // one thread per 16 bytes of the output; the grid holds 2^31 - 1 blocks of 256
    const long long per_tile = (long long)((K / 2 + 127) / 128) * 2048, tiles = (long long)E * n_tiles;
    if (tiles > ((1ll << 39) - 256) / per_tile) return HK_ERR_BAD_SHAPE;
    const long long total = tiles * per_tile;
    hipLaunchKernelGGL(moe_preshuffle_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint8_t*)w, (const uint8_t*)scales, E, N, K, scale_pitch, mode,
                       n_tiles, (uint8_t*)out_w, (uint8_t*)out_s);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// Workspace layout of hk_moe_mxfp4_forward (all regions 256-byte aligned).
struct MoeWs {
    size_t ids, w, sorted, offsets, inv, sort_ws, items1, items2, nitems, xq, xs, hq, hs, o, total;
    int max_items1, max_items2;
};
static MoeWs moe_ws_layout(int T, int H, int I, int E, int k, bool a8 = false) {
    MoeWs L;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t at = off; off = (off + bytes + 255) / 256 * 256; return at; };
    const size_t S = (size_t)T * k;
    L.ids = take(S * 4); L.w = take(S * 4); L.sorted = take(S * 4); L.offsets = take((size_t)(E + 1) * 4);
    L.inv = take(S * 4); L.sort_ws = take(hk_moe_sort_workspace_bytes(T, k, E));
    const int max_tiles = (int)(S / kMoeBM) + E;
    L.max_items1 = max_tiles * ((I + 127) / 128);
    L.max_items2 = max_tiles * ((H + 255) / 256);
    L.items1 = take((size_t)L.max_items1 * sizeof(MoeItem));
    L.items2 = take((size_t)L.max_items2 * sizeof(MoeItem));
    L.nitems = take(8);
    const size_t nk1 = (H / 2 + 127) / 128, nk2 = (I / 2 + 127) / 128;  // K-step-major activation tiles
    const size_t row = a8 ? 256 : 128;  // activation bytes per row and K-step
    L.xq = take(nk1 * S * row); L.xs = take(std::max(nk1 * S * 8, (nk1 + 15) / 16 * (size_t)T * 128));
    L.hq = take(nk2 * S * row); L.hs = take(nk2 * S * 8);
    L.o = take(S * (size_t)H * 2);
    L.total = off;
    return L;
}

static bool moe_mxfp4_shape_ok(int T, int H, int I, int E, int k);
// (0 for a shape the entry points refuse)
extern "C" size_t hk_moe_mxfp4_workspace_bytes(int T, int H, int I, int E, int k) {
    if (!moe_mxfp4_shape_ok(T, H, I, E, k)) return 0;
    return moe_ws_layout(T, H, I, E, k).total;
}
extern "C" size_t hk_moe_mxfp4_a8_workspace_bytes(int T, int H, int I, int E, int k) {
    if (!moe_mxfp4_shape_ok(T, H, I, E, k)) return 0;
    if ((long long)T * k * (((long long)H + 255) / 256 * 256) >= (1ll << 31) ||
        (long long)T * k * (((long long)I + 255) / 256 * 256) >= (1ll << 31))
        return 0;   // MXFP8 rows are twice as long
    return moe_ws_layout(T, H, I, E, k, true).total;
}

// The shapes the layer's kernels address with 32-bit offsets.
static bool moe_mxfp4_shape_ok(int T, int H, int I, int E, int k) {
    if (T <= 0 || E <= 0 || k <= 0 || k > E || k > 64 || E > 512) return false;
    if (H <= 0 || I <= 0 || (H % 32) != 0 || (I % 32) != 0) return false;
    return (long long)T * k < (1ll << 24) && (long long)T * k * (((I / 2 + 127) / 128) * 128) < (1ll << 31) &&
           (long long)T * k * (((H / 2 + 127) / 128) * 128) < (1ll << 31) && (long long)2 * I * (H / 2) < (1ll << 31) &&
           (long long)H * (I / 2) < (1ll << 31);
}
static int moe_mxfp4_check(int T, int H, int I, int E, int k, int w13_scale_pitch, int w2_scale_pitch) {
    if (!moe_mxfp4_shape_ok(T, H, I, E, k)) return HK_ERR_BAD_SHAPE;
    if (w13_scale_pitch < H / 32 || (w13_scale_pitch % 8) != 0 || w2_scale_pitch < I / 32 ||
        (w2_scale_pitch % 8) != 0)
        return HK_ERR_BAD_SHAPE;
    return HK_OK;
}

static MoeBuildItems moe_items_args(uint8_t* ws, const MoeWs& L, int I, int H, bool a8, int weight_layout, bool gather) {
    MoeBuildItems b;
    b.bm = a8 ? (gather ? S4Cfg<true, true>::kBM : S4Cfg<true, false>::kBM) : weight_layout ? kStBM : kMoeBM;
    b.items[0] = (MoeItem*)(ws + L.items1); b.items[1] = (MoeItem*)(ws + L.items2);
    b.n_tiles[0] = (I + 127) / 128; b.n_tiles[1] = (H + 255) / 256;
    return b;
}
static MxQuantizeArgs moe_quantize_args(const void* x_bf16, const int32_t* sorted_slots, const int32_t* slot_to_pos,
                                        int k, int T, int H, int I, uint8_t* ws, const MoeWs& L) {
    MxQuantizeArgs a;
    a.x = (const uint16_t*)x_bf16; a.sorted_slots = sorted_slots; a.slot_to_pos = slot_to_pos;
    a.topk = k; a.T = T; a.cols = H;
    a.tiled = ws + L.xq; a.tiled_scales = ws + L.xs; a.tiled2 = ws + L.hq; a.tiled2_scales = ws + L.hs;
    a.K2 = I;
    return a;
}
// Whether the layer's gate+up kernel gathers its activation rows by token (the 4-wave streaming
// kernel with the plain epilogue): x is then quantized once per token; the other kernels take it
// permuted into sorted order, one row per slot.
// It pays while the quantized x stays in an XCD's L2 next to the weight stream (measured: up to
// 4096 tokens of 2880 MXFP4 columns, 1024 of MXFP8).
static bool moe_gathers(int weight_layout, bool ext, bool a8, int T, int H) {
    return weight_layout == 1 && !ext && (long long)T * H * (a8 ? 2 : 1) <= 12ll << 20;
}

// Every argument check of the expert MLP, made before the first launch of a call (the forward entry points run
// top-k, sort and quantization in front of the expert GEMMs: a call that is going to be refused must not have
// started any of them).
static int moe_mxfp4_validate(const void* x_bf16, const void* w13, const void* w13_scales, int w13_scale_pitch,
                              const void* w2, const void* w2_scales, int w2_scale_pitch, const void* y_bf16, int T,
                              int H, int I, int E, int k, int weight_layout, const float* bias13, const float* bias2,
                              int activation, float limit, const void* workspace, size_t workspace_bytes, bool a8) {
    if (activation != 0 && activation != 1) return HK_ERR_UNSUPPORTED;
    if (a8 && weight_layout != 1) return HK_ERR_UNSUPPORTED;
    if (activation == 1 && !(limit > 0.f)) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)bias13 | (uintptr_t)bias2) & 15u) return HK_ERR_BAD_ALIGNMENT;
    // the bias arrays are addressed with 32-bit byte offsets
    if ((bias13 && (unsigned long long)E * 2 * I * 4 >= (1ull << 32)) || (bias2 && (unsigned long long)E * H * 4 >= (1ull << 32)))
        return HK_ERR_BAD_SHAPE;
    if (!x_bf16 || !w13 || !w13_scales || !w2 || !w2_scales || !y_bf16) return HK_ERR_NULL_POINTER;
    if (weight_layout != 0 && weight_layout != 1) return HK_ERR_UNSUPPORTED;
    const int st = moe_mxfp4_check(T, H, I, E, k, weight_layout ? moe_round_up(H / 32, 8) : w13_scale_pitch,
                                   weight_layout ? moe_round_up(I / 32, 8) : w2_scale_pitch);
    if (st != HK_OK) return st;
    // MXFP8 activation tiles are twice as large: their 32-bit buffer offsets must still fit
    if (a8 && ((long long)T * k * ((H + 255) / 256 * 256) >= (1ll << 31) ||
               (long long)T * k * ((I + 255) / 256 * 256) >= (1ll << 31)))
        return HK_ERR_BAD_SHAPE;
    const MoeWs L = moe_ws_layout(T, H, I, E, k, a8);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    if (((uintptr_t)x_bf16 | (uintptr_t)w13 | (uintptr_t)w2 | (uintptr_t)y_bf16 | (uintptr_t)workspace) & 15u)
        return HK_ERR_BAD_ALIGNMENT;
    if (((uintptr_t)w13_scales | (uintptr_t)w2_scales) & 3u) return HK_ERR_BAD_ALIGNMENT;
    return HK_OK;
}

// Expert MLP on already routed and sorted tokens (steps 3-6 of the forward pass). a8: MXFP8
// activations (pre-shuffled weights only).
static int moe_mxfp4_experts_impl(const void* x_bf16, const void* w13, const void* w13_scales,
                                  int w13_scale_pitch, const void* w2, const void* w2_scales,
                                  int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                                  const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                  int T, int H, int I, int E, int k, int weight_layout,
                                  const float* bias13, const float* bias2, int activation, float alpha,
                                  float limit, int w13_interleaved, void* workspace,
                                  size_t workspace_bytes, void* stream, bool a8, bool x_quantized = false) {
    if (!topk_w || !sorted_slots || !expert_offsets || !slot_to_pos) return HK_ERR_NULL_POINTER;
    int st = moe_mxfp4_validate(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch, y_bf16, T, H,
                                I, E, k, weight_layout, bias13, bias2, activation, limit, workspace, workspace_bytes,
                                a8);
    if (st != HK_OK) return st;
    const bool ext = bias13 || bias2 || activation != 0 || w13_interleaved;
    const MoeWs L = moe_ws_layout(T, H, I, E, k, a8);
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    const int S = T * k;

    int32_t* nitems = (int32_t*)(ws + L.nitems);
    const bool gather = moe_gathers(weight_layout, ext, a8, T, H);
    // non-temporal weight loads while most experts' rows fit one work item (their weights are then read
    // once): mean + one standard deviation of the rows per expert under uniform routing
    const bool nt = moe_rows_fit_one_item(T, k, E, a8 ? (gather ? S4Cfg<true, true>::kBM : S4Cfg<true, false>::kBM) : kStBM);
    if (!x_quantized) {   // (the forward pass of a small layer has done this in its sort launch)
        const int nk1 = (H / 2 + 127) / 128;
        const MoeBuildItems b = moe_items_args(ws, L, I, H, a8, weight_layout, gather);
        const MxQuantizeArgs qa = moe_quantize_args(x_bf16, sorted_slots, slot_to_pos, k, T, H, I, ws, L);
        auto qp = a8 ? (gather ? mx_quantize_permute_kernel<true, false> : mx_quantize_permute_kernel<true, true>)
                     : (gather ? mx_quantize_permute_kernel<false, false> : mx_quantize_permute_kernel<false, true>);
        hipLaunchKernelGGL(qp, dim3((T + kQpRows - 1) / kQpRows + 2, (nk1 + 3) / 4), dim3(128), 0, s, qa,
                           expert_offsets, E, b, nitems);
    }

    MoeGemmParams p{};
    p.A = ws + L.xq; p.SA = ws + L.xs; p.S = S;
    p.row_slots = gather ? sorted_slots : nullptr; p.a_rows = gather ? T : S;
    p.topk_magic = k == 1 ? 0u : (uint32_t)(((1ull << 32) + (uint64_t)k - 1) / (uint64_t)k);
    p.B = (const uint8_t*)w13; p.SB = (const uint8_t*)w13_scales;
    p.b_pitch = H / 2; p.sb_pitch = w13_scale_pitch;
    p.b_expert_stride = (long long)2 * I * (H / 2); p.sb_expert_stride = (long long)2 * I * w13_scale_pitch;
    if (weight_layout) {
        const long long tiles = (long long)((I + 127) / 128) * ((H / 2 + 127) / 128);
        p.b_expert_stride = tiles * kMoeBTile; p.sb_expert_stride = tiles * kMoeScaleB;
    }
    p.items = (const MoeItem*)(ws + L.items1); p.num_items = nitems;
    p.out0 = ws + L.hq; p.out_scales = ws + L.hs;
    p.K = H; p.N = I; p.n_tiles_n = (I + 127) / 128;
    p.bias = bias13; p.bias_bytes = (uint32_t)((size_t)E * 2 * I * 4); p.act = activation; p.alpha = alpha; p.limit = limit; p.interleaved = w13_interleaved != 0;
    if (a8)
        st = ext ? launch_moe_stream<0, true, true>(p, L.max_items1, s, nt)
                 : gather ? launch_moe_stream<0, false, true, true>(p, L.max_items1, s, nt)
                          : launch_moe_stream<0, false, true>(p, L.max_items1, s, nt);
    else if (ext)
        st = weight_layout ? launch_moe_stream<0, true, false>(p, L.max_items1, s, nt) : launch_moe_gemm<0, true>(p, L.max_items1, s);
    else
        st = gather ? launch_moe_stream<0, false, false, true>(p, L.max_items1, s, nt)
             : weight_layout ? launch_moe_stream<0, false, false>(p, L.max_items1, s, nt) : launch_moe_gemm<0, false>(p, L.max_items1, s);
    if (st != HK_OK) return st;

    MoeGemmParams q{};
    q.A = ws + L.hq; q.SA = ws + L.hs; q.S = S;
    q.B = (const uint8_t*)w2; q.SB = (const uint8_t*)w2_scales;
    q.b_pitch = I / 2; q.sb_pitch = w2_scale_pitch;
    q.b_expert_stride = (long long)H * (I / 2); q.sb_expert_stride = (long long)H * w2_scale_pitch;
    if (weight_layout) {
        const long long tiles = (long long)((H + 255) / 256) * ((I / 2 + 127) / 128);
        q.b_expert_stride = tiles * kMoeBTile; q.sb_expert_stride = tiles * kMoeScaleB;
    }
    q.items = (const MoeItem*)(ws + L.items2); q.num_items = nitems + 1;
    q.out0 = ws + L.o; q.out_scales = nullptr;
    q.K = I; q.N = H; q.n_tiles_n = (H + 255) / 256;
    q.bias = bias2; q.bias_bytes = (uint32_t)((size_t)E * H * 4);
    if (a8)
        st = bias2 ? launch_moe_stream<1, true, true>(q, L.max_items2, s, nt) : launch_moe_stream<1, false, true>(q, L.max_items2, s, nt);
    else if (bias2)
        st = weight_layout ? launch_moe_stream<1, true, false>(q, L.max_items2, s, nt) : launch_moe_gemm<1, true>(q, L.max_items2, s);
    else
        st = weight_layout ? launch_moe_stream<1, false, false>(q, L.max_items2, s, nt) : launch_moe_gemm<1, false>(q, L.max_items2, s);
    if (st != HK_OK) return st;

    return hk_moe_unpermute(ws + L.o, topk_w, slot_to_pos, T, k, H, y_bf16, stream);
}

extern "C" int hk_moe_mxfp4_experts_ex(const void* x_bf16, const void* w13, const void* w13_scales,
                                       int w13_scale_pitch, const void* w2, const void* w2_scales,
                                       int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                                       const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                       int T, int H, int I, int E, int k, int weight_layout,
                                       const float* bias13, const float* bias2, int activation, float alpha,
                                       float limit, int w13_interleaved, void* workspace,
                                       size_t workspace_bytes, void* stream) {
    return moe_mxfp4_experts_impl(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch, topk_w,
                                  sorted_slots, expert_offsets, slot_to_pos, y_bf16, T, H, I, E, k, weight_layout,
                                  bias13, bias2, activation, alpha, limit, w13_interleaved, workspace,
                                  workspace_bytes, stream, false);
}

extern "C" int hk_moe_mxfp4_a8_experts(const void* x_bf16, const void* w13_shuffled, const void* w13_scales_shuffled,
                                       const void* w2_shuffled, const void* w2_scales_shuffled, const float* topk_w,
                                       const int32_t* sorted_slots, const int32_t* expert_offsets,
                                       const int32_t* slot_to_pos, void* y_bf16, int T, int H, int I, int E, int k,
                                       const float* bias13, const float* bias2, int activation, float alpha,
                                       float limit, int w13_interleaved, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    return moe_mxfp4_experts_impl(x_bf16, w13_shuffled, w13_scales_shuffled, 0, w2_shuffled, w2_scales_shuffled, 0,
                                  topk_w, sorted_slots, expert_offsets, slot_to_pos, y_bf16, T, H, I, E, k, 1, bias13,
                                  bias2, activation, alpha, limit, w13_interleaved, workspace, workspace_bytes, stream,
                                  true);
}

extern "C" int hk_moe_mxfp4_experts(const void* x_bf16, const void* w13, const void* w13_scales,
                                    int w13_scale_pitch, const void* w2, const void* w2_scales,
                                    int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                                    const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                    int T, int H, int I, int E, int k, int weight_layout, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    return hk_moe_mxfp4_experts_ex(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch, topk_w,
                                   sorted_slots, expert_offsets, slot_to_pos, y_bf16, T, H, I, E, k, weight_layout,
                                   nullptr, nullptr, 0, 0.f, 0.f, 0, workspace, workspace_bytes, stream);
}

static int moe_mxfp4_forward_impl(const void* x_bf16, const float* router_logits, const void* w13,
                                  const void* w13_scales, int w13_scale_pitch, const void* w2,
                                  const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H,
                                  int I, int E, int k, int weight_layout, const float* bias13,
                                  const float* bias2, int activation, float alpha, float limit,
                                  int w13_interleaved, void* workspace, size_t workspace_bytes,
                                  void* stream, bool a8) {
    if (!router_logits) return HK_ERR_NULL_POINTER;
    int st = moe_mxfp4_validate(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch, y_bf16, T, H,
                                I, E, k, weight_layout, bias13, bias2, activation, limit, workspace, workspace_bytes,
                                a8);
    if (st != HK_OK) return st;
    const MoeWs L = moe_ws_layout(T, H, I, E, k, a8);
    uint8_t* ws = (uint8_t*)workspace;
    st = hk_moe_topk_softmax(router_logits, T, E, k, (int32_t*)(ws + L.ids), (float*)(ws + L.w), stream);
    if (st != HK_OK) return st;
    const bool ext = bias13 || bias2 || activation != 0 || w13_interleaved;
    bool fused = false;
    if (moe_gathers(weight_layout, ext, a8, T, H) && (long long)T * k <= kSortSmallMax && x_bf16 &&
        (((uintptr_t)x_bf16 | (uintptr_t)workspace) & 15u) == 0) {
        // sort, item lists and the quantization of x in one launch (moe_sort_quantize_kernel)
        const int S = T * k, nchunks = (S + kSortChunk - 1) / kSortChunk;
        const int nk1 = (H / 2 + 127) / 128;
        const MoeBuildItems b = moe_items_args(ws, L, I, H, a8, weight_layout, true);
        const MxQuantizeArgs qa = moe_quantize_args(x_bf16, nullptr, nullptr, k, T, H, I, ws, L);
        const int grid = nchunks + 2 * kFusedItemParts + (T + kQpRows - 1) / kQpRows * ((nk1 + 7) / 8);
        auto kern = a8 ? moe_sort_quantize_kernel<true> : moe_sort_quantize_kernel<false>;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const int32_t*)(ws + L.ids), E,
                           (int32_t*)(ws + L.offsets), (int32_t*)(ws + L.sorted), (int32_t*)(ws + L.inv), qa, b,
                           (int32_t*)(ws + L.nitems));
        if (hipGetLastError() != hipSuccess) return HK_ERR_LAUNCH;
        fused = true;
    } else {
        st = hk_moe_sort((const int32_t*)(ws + L.ids), T, k, E, (int32_t*)(ws + L.sorted), (int32_t*)(ws + L.offsets),
                         (int32_t*)(ws + L.inv), ws + L.sort_ws, hk_moe_sort_workspace_bytes(T, k, E), stream);
        if (st != HK_OK) return st;
    }
    return moe_mxfp4_experts_impl(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch,
                                  (const float*)(ws + L.w), (const int32_t*)(ws + L.sorted),
                                  (const int32_t*)(ws + L.offsets), (const int32_t*)(ws + L.inv), y_bf16, T, H, I,
                                  E, k, weight_layout, bias13, bias2, activation, alpha, limit, w13_interleaved,
                                  workspace, workspace_bytes, stream, a8, fused);
}

extern "C" int hk_moe_mxfp4_forward_ex(const void* x_bf16, const float* router_logits, const void* w13,
                                       const void* w13_scales, int w13_scale_pitch, const void* w2,
                                       const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H,
                                       int I, int E, int k, int weight_layout, const float* bias13,
                                       const float* bias2, int activation, float alpha, float limit,
                                       int w13_interleaved, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    return moe_mxfp4_forward_impl(x_bf16, router_logits, w13, w13_scales, w13_scale_pitch, w2, w2_scales,
                                  w2_scale_pitch, y_bf16, T, H, I, E, k, weight_layout, bias13, bias2, activation,
                                  alpha, limit, w13_interleaved, workspace, workspace_bytes, stream, false);
}

extern "C" int hk_moe_mxfp4_a8_forward(const void* x_bf16, const float* router_logits, const void* w13_shuffled,
                                       const void* w13_scales_shuffled, const void* w2_shuffled,
                                       const void* w2_scales_shuffled, void* y_bf16, int T, int H, int I, int E,
                                       int k, const float* bias13, const float* bias2, int activation, float alpha,
                                       float limit, int w13_interleaved, void* workspace, size_t workspace_bytes,
                                       void* stream) {
    return moe_mxfp4_forward_impl(x_bf16, router_logits, w13_shuffled, w13_scales_shuffled, 0, w2_shuffled,
                                  w2_scales_shuffled, 0, y_bf16, T, H, I, E, k, 1, bias13, bias2, activation, alpha,
                                  limit, w13_interleaved, workspace, workspace_bytes, stream, true);
}

extern "C" int hk_moe_mxfp4_forward(const void* x_bf16, const float* router_logits, const void* w13,
                                    const void* w13_scales, int w13_scale_pitch, const void* w2,
                                    const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H, int I,
                                    int E, int k, int weight_layout, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    return hk_moe_mxfp4_forward_ex(x_bf16, router_logits, w13, w13_scales, w13_scale_pitch, w2, w2_scales,
                                   w2_scale_pitch, y_bf16, T, H, I, E, k, weight_layout, nullptr, nullptr, 0, 0.f,
                                   0.f, 0, workspace, workspace_bytes, stream);
}
