// FP8 block-scaled fused MoE for gfx950 (DeepSeek-V3 style quantization): activations e4m3 with
// one fp32 scale per 1 x 128 block, weights e4m3 with one fp32 scale per 128 x 128 block.
//
// The reference has no MoE code (no counterpart to cite). Structure as in the MXFP4 MoE of this
// library (moe_mxfp4.hip): persistent 8-wave workgroups walk a device-built list of (m-tile,
// n-tile) work items, operands stream through a three-stage LDS ring with direct global->LDS
// loads, activations live in K-step-major tiles. fp32 block scales cannot ride the MFMA's scale
// port (e8m0 only), so every K-step of 128 is one unscaled v_mfma_f32_16x16x128_f8f6f4 into a
// fresh accumulator that a VALU FMA folds into the running sum:
//     acc += partial * (x_scale[row, kb] * w_scale[col / 128, kb]).
#include "moe_common.h"
#include "../../include/hk355.h"

namespace hk {

typedef __attribute__((address_space(3))) const float lds_f32_t;
typedef __attribute__((address_space(3))) float lds_f32_mut_t;
typedef __attribute__((address_space(3))) const v4f lds_v4f_t;

constexpr float kE4m3Max = 448.0f;

// Two floats -> two e4m3 bytes (bits [15:0]), round to nearest even, saturating at +-448.
__device__ __forceinline__ uint32_t cvt2_e4m3(float a, float b) {
    a = __builtin_amdgcn_fmed3f(a, -kE4m3Max, kE4m3Max);
    b = __builtin_amdgcn_fmed3f(b, -kE4m3Max, kE4m3Max);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}
// scale of a block with maximum magnitude amax: amax / 448, or 1 for an all-zero block
__device__ __forceinline__ float e4m3_block_scale(float amax) {
    return amax > 0.f ? __fdiv_rn(amax, kE4m3Max) : 1.0f;
}
__device__ __forceinline__ v2i quant8_e4m3(const float (&v)[8], float s) {
    v2i out;
    out.x = (int)(cvt2_e4m3(__fdiv_rn(v[0], s), __fdiv_rn(v[1], s)) |
                  (cvt2_e4m3(__fdiv_rn(v[2], s), __fdiv_rn(v[3], s)) << 16));
    out.y = (int)(cvt2_e4m3(__fdiv_rn(v[4], s), __fdiv_rn(v[5], s)) |
                  (cvt2_e4m3(__fdiv_rn(v[6], s), __fdiv_rn(v[7], s)) << 16));
    return out;
}

// x [rows, cols] bf16 -> e4m3 [rows, cols] + fp32 scales [rows, cols / 128] (1 x 128 blocks).
// One thread per 8 elements, 16 threads per block.
__global__ __launch_bounds__(256) void fp8_quantize_rows_1x128_kernel(const uint16_t* __restrict__ x, int rows,
                                                                      int cols, uint8_t* __restrict__ q,
                                                                      float* __restrict__ scales) {
    const int per_row = cols / 8;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const int row = (int)(gid / per_row), c8 = (int)(gid % per_row);
    if (row >= rows) return;
    const v4i raw = *(const v4i*)(x + (size_t)row * cols + c8 * 8);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float((uint32_t)raw[i] << 16);
        v[2 * i + 1] = __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float s = e4m3_block_scale(amax);
    *(v2i*)(q + (size_t)row * cols + c8 * 8) = quant8_e4m3(v, s);
    if ((c8 & 15) == 0) scales[(size_t)row * (cols / 128) + (c8 >> 4)] = s;
}

// Permute quantized activations into K-step-major tiles in sorted order: row `pos` of the output
// is token sorted_slots[pos] / topk. tiled [nk][S][128] bytes, tiled_scales [nk][S] floats.
__global__ __launch_bounds__(256) void fp8blk_permute_kernel(const uint8_t* __restrict__ xq,
                                                             const float* __restrict__ xs,
                                                             const int32_t* __restrict__ sorted_slots, int topk,
                                                             int S, int cols, uint8_t* __restrict__ tiled,
                                                             float* __restrict__ tiled_scales) {
    const int per_row = cols / 16;  // 16-byte chunks
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    const int pos = (int)(gid / per_row), c = (int)(gid % per_row);
    if (pos >= S) return;
    const int row = sorted_slots[pos] / topk;
    const size_t tile_row = (size_t)(c >> 3) * S + pos;
    *(v4i*)(tiled + tile_row * 128 + (c & 7) * 16) = *(const v4i*)(xq + (size_t)row * cols + c * 16);
    if ((c & 7) == 0) tiled_scales[tile_row] = xs[(size_t)row * (cols / 128) + (c >> 3)];
}

struct MoeFp8Params {
    const uint8_t* A;      // activations, K-step-major tiles [nk][S][128] e4m3
    const float* SA;       // their scales [nk][S]
    const uint8_t* B;      // expert weights [E][rows_b][K] e4m3
    const float* SB;       // their scales [E][rows_b / 128][K / 128]
    const MoeItem* items;
    const int32_t* num_items;
    void* out0;            // MODE 0: h as tiles [I / 128][S][128] e4m3; MODE 1: bf16 o [S][N]
    float* out_scales;     // MODE 0: scales of h [I / 128][S]
    long long b_expert_stride, sb_expert_stride;  // bytes / floats
    int K, N, S, n_tiles_n;
};

constexpr int kF8ATile = kMoeBM * 128;             // 16 KiB
constexpr int kF8BTile = 256 * 128;                // 32 KiB
constexpr int kF8Stage = kF8ATile + kF8BTile;      // 48 KiB
constexpr int kF8ScaleBase = 3 * kF8Stage;         // A scales: 3 stages x kMoeBM floats
constexpr int kF8XchBase = kF8ScaleBase + 3 * kMoeBM * 4;  // epilogue exchange: kMoeBM x 4 floats
constexpr int kF8Lds = kF8XchBase + kMoeBM * 16;

// dword global->LDS load restricted to the lanes in `mask` (lane l lands at lds_base + 4*l)
__device__ __forceinline__ void dma4_lanes(v4i srd, uint32_t lds_base, uint32_t voff, uint32_t soff,
                                           uint64_t mask) {
    uint64_t saved;
    asm volatile(
        "s_mov_b64 %0, exec\n\t"
        "s_mov_b64 exec, %5\n\t"
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "buffer_load_dword %2, %3, %4 offen lds\n\t"
        "s_mov_b64 exec, %0"
        : "=&s"(saved)
        : "s"(lds_base), "v"(voff), "s"(srd), "s"(soff), "s"(mask)
        : "memory", "m0");
}

struct MoeFp8Addr {
    v4i srd_b;
    uint32_t voff_b[4];
    const float* sb0;  // weight scales of the first row block this wave needs, K-step 0
    const float* sb1;  // MODE 0: scales of the up-projection row block
    int row_start, rows, n0, n_tile;
    bool valid;
};

template <int MODE>
__global__ __launch_bounds__(512) void moe_fp8blk_gemm_kernel(const MoeFp8Params p) {
    constexpr int NW = 8, MT = kMoeBM / 32, NT = 4, NA = kMoeBM / 64;
    constexpr int kDma = NA + 4 + 1;
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    const int lane = lane_id(), w = wave_id();
    const int wm = w >> 2, wn = w & 3;

    const int n_items = scalar_load_x1(p.num_items);
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int it_stride = ((int)gridDim.x - xcd + kNumXcd - 1) / kNumXcd;
    const int per_xcd = (n_items + kNumXcd - 1) / kNumXcd;
    int it = xcd * per_xcd + slot;
    const int it_end = min(n_items, (xcd + 1) * per_xcd);
    if (it >= it_end) return;

    const int nk = p.K >> 7;
    const int rows_b = MODE == 0 ? 2 * p.N : p.N;
    const v4i srd_a = make_srd(p.A, (uint32_t)nk * (uint32_t)p.S * 128u);
    const v4i srd_sa = make_srd(p.SA, (uint32_t)nk * (uint32_t)p.S * 4u);
    const uint32_t chunk16 = swz_chunk(8 * w + (lane >> 3), lane & 7);

    auto make_addr = [&](int idx, MoeFp8Addr& a) {
        a.valid = idx < it_end;
        if (!a.valid) idx = it_end - 1;
        const v4i item = scalar_load_x4(p.items + idx);
        const int expert = item.x;
        a.row_start = item.y;
        a.rows = item.z;
        a.n_tile = item.w;
        a.n0 = a.n_tile * (MODE == 0 ? 128 : 256);
        a.srd_b = make_srd(p.B + (size_t)expert * p.b_expert_stride, (uint32_t)rows_b * (uint32_t)p.K);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            a.voff_b[i] = (uint32_t)moe_b_row(MODE, 8 * (i * NW + w) + (lane >> 3), a.n_tile, p.N) * (uint32_t)p.K +
                          chunk16 * 16u;
        const float* sb = p.SB + (size_t)expert * p.sb_expert_stride;
        if (MODE == 0) {
            a.sb0 = sb + (size_t)a.n_tile * nk;                    // gate rows n0 .. n0+127
            a.sb1 = sb + (size_t)(p.N / 128 + a.n_tile) * nk;      // up rows I + n0 ..
        } else {
            a.sb0 = sb + (size_t)min(2 * a.n_tile + (wn >> 1), p.N / 128 - 1) * nk;
            a.sb1 = a.sb0;
        }
    };

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kF8ScaleBase + (uint32_t)w * (kMoeBM / 8) * 4u);
    uint32_t voff_a[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) voff_a[i] = (uint32_t)(8 * (i * NW + w) + (lane >> 3)) * 128u + chunk16 * 16u;
    const uint32_t voff_sa = (uint32_t)((w * (kMoeBM / 8) + lane) * 4);
    constexpr uint64_t kSaMask = (1ull << (kMoeBM / 8)) - 1ull;

    auto issue_tile = [&](const MoeFp8Addr& a, int stage, int kt) {
        v4i sa = srd_a, sb = a.srd_b, ssa = srd_sa;
        if (!a.valid || kt >= nk) { sa.z = 0; sb.z = 0; ssa.z = 0; }
        const uint32_t row_base = (uint32_t)kt * (uint32_t)p.S + (uint32_t)a.row_start;
        const uint32_t dst = lds_wave + (uint32_t)stage * kF8Stage;
#pragma unroll
        for (int i = 0; i < NA; ++i) dma16(sa, dst + i * NW * 1024, voff_a[i], row_base * 128u);
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(sb, dst + kF8ATile + i * NW * 1024, a.voff_b[i], (uint32_t)kt * 128u);
        dma4_lanes(ssa, lds_sa_wave + (uint32_t)stage * (kMoeBM * 4), voff_sa, row_base * 4u, kSaMask);
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    const uint32_t a_lo0 = lds0 + wm * 2048 + rd_lo, a_hi0 = lds0 + wm * 2048 + rd_hi;
    const uint32_t b_lo0 = lds0 + kF8ATile + wn * (64 * 128) + rd_lo;
    const uint32_t b_hi0 = lds0 + kF8ATile + wn * (64 * 128) + rd_hi;
    const uint32_t sa_rd0 = lds0 + kF8ScaleBase + (wm * 16 + r) * 4u;

    v4f acc[MT][NT];
    MoeFp8Addr cur, nxt;

    // One K-step (= one 128-wide scale block) on LDS stage st.
    auto compute = [&](int st, int rows, int kt) {
        uint32_t a_lo = a_lo0 + (uint32_t)st * kF8Stage, a_hi = a_hi0 + (uint32_t)st * kF8Stage;
        uint32_t b_lo = b_lo0 + (uint32_t)st * kF8Stage, b_hi = b_hi0 + (uint32_t)st * kF8Stage;
        uint32_t sa_rd = sa_rd0 + (uint32_t)st * (kMoeBM * 4);
        asm volatile("" : "+v"(a_lo), "+v"(a_hi), "+v"(b_lo), "+v"(b_hi), "+v"(sa_rd));
        const float ws0 = __int_as_float(scalar_load_x1(cur.sb0 + kt));
        const float ws1 = MODE == 0 ? __int_as_float(scalar_load_x1(cur.sb1 + kt)) : ws0;
        v8i bf[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) bf[n] = lds_frag(b_lo, b_hi, n * 2048);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (16 * (2 * m + wm) < rows) {
                const v8i af = lds_frag(a_lo, a_hi, m * 4096);
                const float xs = *(lds_f32_t*)(uintptr_t)(sa_rd + m * 128);
                const float s0 = xs * ws0, s1 = xs * ws1;
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    const v4f part = mfma_fp8_16x16x128(bf[n], af, v4f{0.f, 0.f, 0.f, 0.f});
                    const float sc = (n & 1) ? s1 : s0;  // MODE 0: odd tiles are up-projection rows
                    acc[m][n] += part * sc;
                }
            }
        }
    };

    auto epilogue = [&](const MoeFp8Addr& a) {
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
                    if (col + 8 > p.N) continue;
                    const v4f x = acc[m][2 * q], y = acc[m][2 * q + 1];
                    v4i o4;
                    o4.x = pack_bf16(x.x, x.y); o4.y = pack_bf16(x.z, x.w);
                    o4.z = pack_bf16(y.x, y.y); o4.w = pack_bf16(y.z, y.w);
                    *(v4i*)(out + pos * p.N + col) = o4;
                }
            }
        } else {
            // h = silu(gate) * up for this wave's 32 of the tile's 128 h columns; the tile's 128
            // columns are one 1 x 128 quantization block, so the row maxima of the four column
            // waves are combined through LDS.
            uint8_t* hq = (uint8_t*)p.out0;
            float h[MT][8];
            const uint32_t xch = lds0 + kF8XchBase;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const v4f gt = acc[m][2 * q], up = acc[m][2 * q + 1];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float gv = gt[j];
                        h[m][4 * q + j] = gv / (1.0f + __expf(-gv)) * up[j];
                    }
                }
                float amax = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[m][i]));
                amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                const int row = 16 * (2 * m + wm) + (int)r;
                if (g == 0) *(lds_f32_mut_t*)(uintptr_t)(xch + (row * 4 + wn) * 4) = amax;
            }
            __syncthreads();
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * (2 * m + wm) + (int)r;
                const v4f am = *(lds_v4f_t*)(uintptr_t)(xch + row * 16);
                const float s = e4m3_block_scale(fmaxf(fmaxf(am.x, am.y), fmaxf(am.z, am.w)));
                if (row < rows) {
                    const size_t tile_row = (size_t)a.n_tile * p.S + (size_t)(row_start + row);
                    *(v2i*)(hq + tile_row * 128 + 32 * wn + 8 * g) = quant8_e4m3(h[m], s);
                    if (wn == 0 && g == 0) p.out_scales[tile_row] = s;
                }
            }
        }
    };

    const int depth = nk >= 2 ? 2 : 1;
    int st = 0;
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
            if (depth == 2) wait_vmcnt<kDma>(); else wait_vmcnt<0>();
            block_barrier();
            const int ahead = kt + depth;
            int stage_ahead = st + depth;
            if (stage_ahead >= 3) stage_ahead -= 3;
            if (ahead < nk) issue_tile(cur, stage_ahead, ahead);
            else issue_tile(nxt, stage_ahead, ahead - nk);
            compute(st, cur.rows, kt);
            st = st == 2 ? 0 : st + 1;
        }
        epilogue(cur);
        it += it_stride;
        if (it >= it_end) break;
        cur = nxt;
    }
    wait_vmcnt<0>();
}

template <int MODE>
static int launch_fp8blk_gemm(const MoeFp8Params& p, int max_items, hipStream_t s) {
    auto kern = moe_fp8blk_gemm_kernel<MODE>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kF8Lds) != hipSuccess)
            return HK_ERR_LAUNCH;
        configured = true;
    }
    const int grid = min(max_items, moe_num_compute_units());
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kF8Lds, s, p);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// ------------------------------------------------------- grouped GEMM, pre-shuffled weights
// Pre-shuffled weight layout: for every (expert, n-tile of 256 tile rows, K-step of 128) one
// contiguous 32 KiB block; inside it, wave by wave (wave wn = tile rows [64 wn, +64)), the wave's
// four MFMA B fragments, each as two 1 KiB pieces in lane order: lane l's 16 bytes of piece
// `part` are tile row 64 wn + 16 f + l % 16 (moe_b_row gives the weight row), K bytes
// 128 kt + 64 part + 16 (l / 16) .. +16. Scales stay in their plain [E][rows/128][K/128] layout.
//   out_w [E][n_tiles][nk][4][4][2][64][16] bytes
__global__ __launch_bounds__(256) void moe_fp8blk_preshuffle_kernel(const uint8_t* __restrict__ w, int E, int N,
                                                                    int K, int mode, int n_tiles,
                                                                    uint8_t* __restrict__ out_w) {
    const int nk = K >> 7;
    const int rows_b = mode == 0 ? 2 * N : N;
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;  // one 16-byte chunk each
    const long long total = (long long)E * n_tiles * nk * 2048;
    if (gid >= total) return;
    const int l = (int)(gid & 63), part = (int)((gid >> 6) & 1), f = (int)((gid >> 7) & 3), wn = (int)((gid >> 9) & 3);
    long long rest = gid >> 11;
    const int kt = (int)(rest % nk); rest /= nk;
    const int nt = (int)(rest % n_tiles);
    const int e = (int)(rest / n_tiles);
    const int row = moe_b_row(mode, 64 * wn + 16 * f + (l & 15), nt, N);
    const int kb = kt * 128 + 64 * part + 16 * (l >> 4);
    *(v4i*)(out_w + gid * 16) = *(const v4i*)(w + ((size_t)e * rows_b + row) * K + kb);
}

// Weight-streaming variant of moe_fp8blk_gemm_kernel for the pre-shuffled layout; same design as
// moe_mxfp4_stream_kernel (moe_mxfp4.hip): 4-wave workgroups, two per CU, wave wn owns weight
// rows [64 wn, +64) x all 128 activation rows; weights go from HBM straight into MFMA operand
// registers two K-steps ahead (a ring of four half-K-step register sets, here the two halves of
// a K-step are its fragment pairs 0,1 and 2,3), only the activation tile passes through a
// four-stage LDS ring. The weights' 128 x 128 block scales ride the same stream as broadcast
// dword loads. Every vector-memory operation is inline asm and counted by hand (see the MXFP4
// kernel for the wait scheme). Results are bit-identical to moe_fp8blk_gemm_kernel.
// Meant for shapes with few rows per expert, where reading the weights once is what counts; with
// hundreds of rows per expert the LDS-staged kernel above overlaps its MFMA work better.
constexpr int kFsStages = 4;
constexpr int kFsStage = kF8ATile + 1024;            // 16 KiB tile + 512 B of row scales (1 KiB slot)
constexpr int kFsXch = kFsStages * kFsStage;         // epilogue exchange: kMoeBM x 4 floats
constexpr int kFsLds = kFsXch + kMoeBM * 16;         // 70 KiB

template <int MODE>
__global__ __launch_bounds__(256, 2) void moe_fp8blk_stream_kernel(const MoeFp8Params p) {
    constexpr int MT = kMoeBM / 16, NT = 4;
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    const int lane = lane_id(), w = wave_id();
    const int n_items = scalar_load_x1(p.num_items);
    const int xcd = blockIdx.x % kNumXcd, slot = blockIdx.x / kNumXcd;
    const int it_stride = ((int)gridDim.x - xcd + kNumXcd - 1) / kNumXcd;
    const int per_xcd = (n_items + kNumXcd - 1) / kNumXcd;
    const int it0 = xcd * per_xcd + slot;
    const int it_end = min(n_items, (xcd + 1) * per_xcd);
    if (it0 >= it_end) return;

    const int nk = p.K >> 7;
    const v4i srd_a = make_srd(p.A, (uint32_t)nk * (uint32_t)p.S * 128u);
    const v4i srd_sa = make_srd(p.SA, (uint32_t)nk * (uint32_t)p.S * 4u);

    struct Cursor { int it, kt, expert, row_start, rows, n_tile; bool valid; };
    auto load_item = [&](Cursor& c) __attribute__((always_inline)) {
        c.valid = c.it < it_end;
        const v4i item = scalar_load_x4(p.items + (c.valid ? c.it : it_end - 1));
        c.expert = item.x; c.row_start = item.y; c.rows = item.z; c.n_tile = item.w;
    };
    auto advance = [&](Cursor& c) __attribute__((always_inline)) {
        if (++c.kt == nk) { c.kt = 0; c.it += it_stride; load_item(c); }
    };
    Cursor cc{it0, 0}, ca{it0, 0}, cb{it0, 0};  // compute, activation fetch, weight fetch
    load_item(cc);
    ca = cc; cb = cc;

    // ---- activation tile: global -> LDS ---------------------------------------------------------
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kF8ATile + (uint32_t)w * 128u);
    const uint32_t chunk16 = swz_chunk(8 * w + (lane >> 3), lane & 7);
    uint32_t voff_a[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) voff_a[i] = (uint32_t)(8 * (i * 4 + w) + (lane >> 3)) * 128u + chunk16 * 16u;
    const uint32_t voff_sa = (uint32_t)(w * 128 + lane * 16);
    // 5 loads: the wave's quarter of the tile (rows 8(4i + w) .. +8) and of its row scales (32 rows)
    auto issue_a = [&](const Cursor& c, int stage) __attribute__((always_inline)) {
        v4i sa = srd_a, ssa = srd_sa;
        if (!c.valid) { sa.z = 0; ssa.z = 0; }
        const uint32_t row_base = (uint32_t)c.kt * (uint32_t)p.S + (uint32_t)c.row_start;
        const uint32_t dst = lds_wave + (uint32_t)stage * kFsStage;
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(sa, dst + i * 4096, voff_a[i], row_base * 128u);
        dma16_lanes(ssa, lds_sa_wave + (uint32_t)stage * kFsStage, voff_sa, row_base * 4u, 0xffull);
    };

    // ---- weights and their block scales: global -> registers -------------------------------------
    const uint32_t voff_b = lane * 16;
    auto srd_b = [&](const Cursor& c) __attribute__((always_inline)) {
        return make_srd(p.B + (size_t)c.expert * p.b_expert_stride + (size_t)c.n_tile * nk * kF8BTile,
                        c.valid ? (uint32_t)nk * kF8BTile : 0u);
    };
    // scale rows of the wave's fragments: MODE 0 gate block n_tile and up block I/128 + n_tile
    // (even fragments are gate rows, odd ones up rows); MODE 1 the 128-row block of the wave's 64 rows
    auto srd_s = [&](const Cursor& c, int which) __attribute__((always_inline)) {
        const float* sb = p.SB + (size_t)c.expert * p.sb_expert_stride;
        int blk;
        if (MODE == 0) blk = which ? p.N / 128 + c.n_tile : c.n_tile;
        else blk = min(2 * c.n_tile + (w >> 1), p.N / 128 - 1);
        return make_srd(sb + (size_t)blk * nk, c.valid ? (uint32_t)nk * 4u : 0u);
    };
    v4i bw[2][2][4];   // [K-step parity][fragment pair][fragment of the pair x 16-byte piece]
    float wsc[2][2];   // [K-step parity][gate / up] block scales of the fetched K-step
    auto load_b_half = [&](const Cursor& c, v4i (&dst)[4], int half) __attribute__((always_inline)) {
        const v4i rs = srd_b(c);
        const uint32_t soff = (uint32_t)c.kt * kF8BTile + (uint32_t)w * 8192u + (uint32_t)half * 4096u;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"
                         : "=v"(dst[j])
                         : "v"(voff_b), "s"(rs), "s"(soff + j * 1024u)
                         : "memory");
    };
    auto load_b_scales = [&](const Cursor& c, float (&dst)[2]) __attribute__((always_inline)) {
        const uint32_t zero = 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const v4i rs = srd_s(c, i);
            asm volatile("buffer_load_dword %0, %1, %2, %3 offen"
                         : "=v"(dst[i])
                         : "v"(zero), "s"(rs), "s"((uint32_t)c.kt * 4u)
                         : "memory");
        }
    };
    auto landed = [&](v4i (&x)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(x[j]));
    };

    // ---- LDS -> registers (activation fragments) ------------------------------------------------
    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = lds0 + r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = lds0 + r * 128u + swz_chunk(r, g + 4) * 16u;
    const uint32_t sa_rd0 = lds0 + kF8ATile + r * 4u;

    v4f acc[MT][NT];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
    };
    // fragment pair `half` (a gate and an up fragment in MODE 0) against all activation fragments
    auto compute_half = [&](int st, int half, int rows, const v4i (&bfr)[4], float ws0, float ws1)
                            __attribute__((always_inline)) {
        uint32_t a_lo = rd_lo + (uint32_t)st * kFsStage, a_hi = rd_hi + (uint32_t)st * kFsStage;
        uint32_t sa_rd = sa_rd0 + (uint32_t)st * kFsStage;
        asm volatile("" : "+v"(a_lo), "+v"(a_hi), "+v"(sa_rd));
        const v8i b0 = __builtin_shufflevector(bfr[0], bfr[1], 0, 1, 2, 3, 4, 5, 6, 7);
        const v8i b1 = __builtin_shufflevector(bfr[2], bfr[3], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (16 * m < rows) {
                const v8i af = lds_frag(a_lo, a_hi, m * 2048);
                const float xs = *(lds_f32_t*)(uintptr_t)(sa_rd + m * 64);
                const float s0 = xs * ws0, s1 = xs * ws1;
                const v4f p0 = mfma_fp8_16x16x128(b0, af, v4f{0.f, 0.f, 0.f, 0.f});
                const v4f p1 = mfma_fp8_16x16x128(b1, af, v4f{0.f, 0.f, 0.f, 0.f});
                acc[m][2 * half] += p0 * s0;
                acc[m][2 * half + 1] += p1 * s1;
            }
        }
    };

    auto epilogue = [&](const Cursor& c) __attribute__((always_inline)) {
        const int rows = c.rows, row_start = c.row_start;
        const int n0 = c.n_tile * (MODE == 0 ? 128 : 256);
        if (MODE == 1) {
            uint16_t* out = (uint16_t*)p.out0;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * m + (int)r;
                if (row >= rows) continue;
                const size_t pos = (size_t)(row_start + row);
#pragma unroll
                for (int q = 0; q < NT / 2; ++q) {
                    const int col = n0 + w * 64 + 32 * q + 8 * (int)g;
                    if (col + 8 > p.N) continue;
                    const v4f x = acc[m][2 * q], y = acc[m][2 * q + 1];
                    v4i o4;
                    o4.x = pack_bf16(x.x, x.y); o4.y = pack_bf16(x.z, x.w);
                    o4.z = pack_bf16(y.x, y.y); o4.w = pack_bf16(y.z, y.w);
                    store_global_b128(out + pos * p.N + col, o4);
                }
            }
        } else {
            // see moe_fp8blk_gemm_kernel: the tile's 128 h columns are one 1 x 128 block, the row
            // maxima of the four waves are combined through LDS
            uint8_t* hq = (uint8_t*)p.out0;
            float h[MT][8];
            const uint32_t xch = lds0 + kFsXch;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const v4f gt = acc[m][2 * q], up = acc[m][2 * q + 1];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float gv = gt[j];
                        h[m][4 * q + j] = gv / (1.0f + __expf(-gv)) * up[j];
                    }
                }
                float amax = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[m][i]));
                amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
                const int row = 16 * m + (int)r;
                if (g == 0) *(lds_f32_mut_t*)(uintptr_t)(xch + (row * 4 + w) * 4) = amax;
            }
            __syncthreads();
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * m + (int)r;
                const v4f am = *(lds_v4f_t*)(uintptr_t)(xch + row * 16);
                const float s = e4m3_block_scale(fmaxf(fmaxf(am.x, am.y), fmaxf(am.z, am.w)));
                if (row < rows) {
                    const size_t tile_row = (size_t)c.n_tile * p.S + (size_t)(row_start + row);
                    store_global_b64(hq + tile_row * 128 + 32 * w + 8 * g, quant8_e4m3(h[m], s));
                    if (w == 0 && g == 0) store_global_b32(p.out_scales + tile_row, __float_as_uint(s));
                }
            }
        }
    };

    // ---- prologue, in the order the K loop issues its loads -------------------------------------
    issue_a(ca, 0); advance(ca);
    issue_a(ca, 1); advance(ca);
    load_b_scales(cb, wsc[0]); load_b_half(cb, bw[0][0], 0); load_b_half(cb, bw[0][1], 1); advance(cb);
    issue_a(ca, 2); advance(ca);
    load_b_scales(cb, wsc[1]); load_b_half(cb, bw[1][0], 0); load_b_half(cb, bw[1][1], 1); advance(cb);
    zero_acc();

    // One stream position. Loads per wave and position, in program order: 5 activation loads
    // (position +3), then 2 scale loads + 4 weight loads after the first fragment pair and 4 weight
    // loads after the second (position +2). Counting the loads issued after the ones needed:
    //   first pair:  4 (second pair) + 15 (previous position)           -> vmcnt(19)
    //   second pair: 15 (previous position) + 5 + 6 (this position)      -> vmcnt(26)
    // A position that ends an item waits for everything but its own 15 loads before it stores
    // (stores share the counter and complete out of order), and the position after it does not wait.
    bool after_stores = false;
    auto step = [&]<int P>(int st) __attribute__((always_inline)) {
        const bool last = cc.valid && cc.kt == nk - 1;
        if (!after_stores) wait_vmcnt<19>();
        block_barrier();
        issue_a(ca, (st + 3) & 3); advance(ca);
        landed(bw[P][0]);
        asm volatile("" : "+v"(wsc[P][0]), "+v"(wsc[P][1]));
        // copies: the scale registers are refilled before the second pair has used them
        float ws0 = wsc[P][0], ws1 = MODE == 0 ? wsc[P][1] : wsc[P][0];
        asm volatile("" : "+v"(ws0), "+v"(ws1));
        const int rows = cc.valid ? cc.rows : 0;
        compute_half(st, 0, rows, bw[P][0], ws0, ws1);
        load_b_scales(cb, wsc[P]);
        load_b_half(cb, bw[P][0], 0);
        if (!after_stores) wait_vmcnt<26>();
        landed(bw[P][1]);
        compute_half(st, 1, rows, bw[P][1], ws0, ws1);
        load_b_half(cb, bw[P][1], 1);
        advance(cb);
        if (last) {
            wait_vmcnt<15>();
            epilogue(cc);
            zero_acc();
        }
        after_stores = last;
        advance(cc);
    };
    for (int st = 0; cc.valid; st ^= 2) {
        step.template operator()<0>(st);
        step.template operator()<1>(st + 1);
    }
    wait_vmcnt<0>();
}

template <int MODE>
static int launch_fp8blk_stream(const MoeFp8Params& p, int max_items, hipStream_t s) {
    auto kern = moe_fp8blk_stream_kernel<MODE>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kFsLds) != hipSuccess)
            return HK_ERR_LAUNCH;
        configured = true;
    }
    const int grid = min(max_items, 2 * moe_num_compute_units());
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), kFsLds, s, p);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

struct Fp8Ws {
    size_t ids, w, sorted, offsets, inv, sort_ws, items1, items2, nitems, xq, xs, hq, hs, o, total;
    int max_items1, max_items2;
};
static Fp8Ws fp8_ws_layout(int T, int H, int I, int E, int k) {
    Fp8Ws L;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t at = off; off = (off + bytes + 255) / 256 * 256; return at; };
    const size_t S = (size_t)T * k;
    L.ids = take(S * 4); L.w = take(S * 4); L.sorted = take(S * 4); L.offsets = take((size_t)(E + 1) * 4);
    L.inv = take(S * 4); L.sort_ws = take(hk_moe_sort_workspace_bytes(T, k, E));
    const int max_tiles = (int)(S / kMoeBM) + E;
    L.max_items1 = max_tiles * (I / 128);
    L.max_items2 = max_tiles * ((H + 255) / 256);
    L.items1 = take((size_t)L.max_items1 * sizeof(MoeItem));
    L.items2 = take((size_t)L.max_items2 * sizeof(MoeItem));
    L.nitems = take(8);
    L.xq = take(S * (size_t)H); L.xs = take(S * (size_t)(H / 128) * 4);
    L.hq = take(S * (size_t)I); L.hs = take(S * (size_t)(I / 128) * 4);
    L.o = take(S * (size_t)H * 2);
    L.total = off;
    return L;
}

static int fp8blk_check(int T, int H, int I, int E, int k) {
    if (T <= 0 || E <= 0 || k <= 0 || k > E || k > 64 || E > 512) return HK_ERR_BAD_SHAPE;
    if (H <= 0 || I <= 0 || (H % 128) != 0 || (I % 128) != 0) return HK_ERR_BAD_SHAPE;
    if ((long long)T * k >= (1ll << 24) || (long long)T * k * H >= (1ll << 32) || (long long)T * k * I >= (1ll << 32) ||
        (long long)2 * I * H >= (1ll << 32))
        return HK_ERR_BAD_SHAPE;
    return HK_OK;
}

}  // namespace hk

using namespace hk;

extern "C" int hk_fp8_quantize_rows_1x128(const void* x_bf16, int rows, int cols, void* q_e4m3, float* scales,
                                          void* stream) {
    if (!x_bf16 || !q_e4m3 || !scales) return HK_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || (cols % 128) != 0) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)x_bf16 | (uintptr_t)q_e4m3) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const long long threads = (long long)rows * (cols / 8);
    hipLaunchKernelGGL(fp8_quantize_rows_1x128_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t*)x_bf16, rows, cols, (uint8_t*)q_e4m3, scales);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" size_t hk_moe_fp8blk_workspace_bytes(int T, int H, int I, int E, int k) {
    if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0) return 0;
    return fp8_ws_layout(T, H, I, E, k).total;
}

extern "C" int hk_moe_fp8blk_preshuffle_bytes(int E, int N, int K, int mode, size_t* w_bytes) {
    if (!w_bytes) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 128) != 0 || (N % 128) != 0 || (mode != 0 && mode != 1))
        return HK_ERR_BAD_SHAPE;
    const size_t n_tiles = mode == 0 ? N / 128 : (N + 255) / 256;
    *w_bytes = (size_t)E * n_tiles * (K / 128) * kF8BTile;
    return HK_OK;
}

extern "C" int hk_moe_fp8blk_preshuffle(const void* w, int E, int N, int K, int mode, void* out_w, void* stream) {
    if (!w || !out_w) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 128) != 0 || (N % 128) != 0 || (mode != 0 && mode != 1))
        return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)w | (uintptr_t)out_w) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const int n_tiles = mode == 0 ? N / 128 : (N + 255) / 256;
    const long long total = (long long)E * n_tiles * (K / 128) * 2048;
    if ((total + 255) / 256 >= (1ll << 31)) return HK_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(moe_fp8blk_preshuffle_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint8_t*)w, E, N, K, mode, n_tiles, (uint8_t*)out_w);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_fp8blk_experts(const void* x_e4m3, const float* x_scales, const void* w13,
                                     const float* w13_scales, const void* w2, const float* w2_scales,
                                     const float* topk_w, const int32_t* sorted_slots, const int32_t* expert_offsets,
                                     const int32_t* slot_to_pos, void* y_bf16, int T, int H, int I, int E, int k,
                                     int weight_layout, void* workspace, size_t workspace_bytes, void* stream) {
    if (!x_e4m3 || !x_scales || !w13 || !w13_scales || !w2 || !w2_scales || !topk_w || !sorted_slots ||
        !expert_offsets || !slot_to_pos || !y_bf16)
        return HK_ERR_NULL_POINTER;
    if (weight_layout != 0 && weight_layout != 1) return HK_ERR_UNSUPPORTED;
    int st = fp8blk_check(T, H, I, E, k);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    if (((uintptr_t)x_e4m3 | (uintptr_t)w13 | (uintptr_t)w2 | (uintptr_t)y_bf16 | (uintptr_t)workspace) & 15u)
        return HK_ERR_BAD_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    const int S = T * k;
    {
        const long long threads = (long long)S * (H / 16);
        hipLaunchKernelGGL(fp8blk_permute_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                           (const uint8_t*)x_e4m3, x_scales, sorted_slots, k, S, H, ws + L.xq, (float*)(ws + L.xs));
    }
    int32_t* nitems = (int32_t*)(ws + L.nitems);
    moe_launch_build_items(expert_offsets, E, I / 128, (MoeItem*)(ws + L.items1), (H + 255) / 256,
                           (MoeItem*)(ws + L.items2), nitems, s);

    MoeFp8Params p{};
    p.A = ws + L.xq; p.SA = (const float*)(ws + L.xs); p.S = S;
    p.B = (const uint8_t*)w13; p.SB = w13_scales;
    p.b_expert_stride = (long long)2 * I * H; p.sb_expert_stride = (long long)(2 * I / 128) * (H / 128);
    p.items = (const MoeItem*)(ws + L.items1); p.num_items = nitems;
    p.out0 = ws + L.hq; p.out_scales = (float*)(ws + L.hs);
    p.K = H; p.N = I; p.n_tiles_n = I / 128;
    if (weight_layout) p.b_expert_stride = (long long)(I / 128) * (H / 128) * kF8BTile;
    st = weight_layout ? launch_fp8blk_stream<0>(p, L.max_items1, s) : launch_fp8blk_gemm<0>(p, L.max_items1, s);
    if (st != HK_OK) return st;

    MoeFp8Params q{};
    q.A = ws + L.hq; q.SA = (const float*)(ws + L.hs); q.S = S;
    q.B = (const uint8_t*)w2; q.SB = w2_scales;
    q.b_expert_stride = (long long)H * I; q.sb_expert_stride = (long long)(H / 128) * (I / 128);
    q.items = (const MoeItem*)(ws + L.items2); q.num_items = nitems + 1;
    q.out0 = ws + L.o; q.out_scales = nullptr;
    q.K = I; q.N = H; q.n_tiles_n = (H + 255) / 256;
    if (weight_layout) q.b_expert_stride = (long long)((H + 255) / 256) * (I / 128) * kF8BTile;
    st = weight_layout ? launch_fp8blk_stream<1>(q, L.max_items2, s) : launch_fp8blk_gemm<1>(q, L.max_items2, s);
    if (st != HK_OK) return st;
    return hk_moe_unpermute(ws + L.o, topk_w, slot_to_pos, T, k, H, y_bf16, stream);
}

extern "C" int hk_moe_fp8blk_forward(const void* x_e4m3, const float* x_scales, const float* router_logits,
                                     const float* router_bias_or_null, int n_group, int topk_group,
                                     float routed_scale, const void* w13, const float* w13_scales, const void* w2,
                                     const float* w2_scales, void* y_bf16, int T, int H, int I, int E, int k,
                                     int weight_layout, void* workspace, size_t workspace_bytes, void* stream) {
    if (!router_logits) return HK_ERR_NULL_POINTER;
    int st = fp8blk_check(T, H, I, E, k);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    uint8_t* ws = (uint8_t*)workspace;
    st = hk_moe_topk_grouped_sigmoid(router_logits, router_bias_or_null, T, E, k, n_group, topk_group, routed_scale,
                                     (int32_t*)(ws + L.ids), (float*)(ws + L.w), stream);
    if (st != HK_OK) return st;
    st = hk_moe_sort((const int32_t*)(ws + L.ids), T, k, E, (int32_t*)(ws + L.sorted), (int32_t*)(ws + L.offsets),
                     (int32_t*)(ws + L.inv), ws + L.sort_ws, hk_moe_sort_workspace_bytes(T, k, E), stream);
    if (st != HK_OK) return st;
    return hk_moe_fp8blk_experts(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, (const float*)(ws + L.w),
                                 (const int32_t*)(ws + L.sorted), (const int32_t*)(ws + L.offsets),
                                 (const int32_t*)(ws + L.inv), y_bf16, T, H, I, E, k, weight_layout, workspace,
                                 workspace_bytes, stream);
}
