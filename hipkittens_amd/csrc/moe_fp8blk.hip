// FP8 block-scaled fused MoE for gfx950 (DeepSeek-V3 style quantization): activations e4m3 with
// one fp32 scale per 1 x 128 block, weights e4m3 with one fp32 scale per 128 x 128 block.
//
// The reference has no MoE code (no counterpart to cite). Structure as in the MXFP4 MoE of this
// library (moe_mxfp4.hip): persistent 8-wave workgroups walk a device-built list of (m-tile,
// n-tile) work items, operands stream through a three-stage LDS ring with direct global->LDS
// loads. The gate+up GEMM fetches its activation rows from the caller's x by token index (no
// permuted copy); the intermediate h lives in K-step-major tiles. fp32 block scales cannot ride the MFMA's scale
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

struct MoeFp8Params {
    const uint8_t* A;      // activations, K-step-major tiles [nk][S][128] e4m3 (GATHER: see below)
    const float* SA;       // their scales [nk][S]
    const uint8_t* B;      // expert weights [E][rows_b][K] e4m3
    const float* SB;       // their scales [E][rows_b / 128][K / 128]
    const MoeItem* items;
    const int32_t* num_items;
    void* out0;            // MODE 0: h as tiles [I / 128][S][128] e4m3; MODE 1: bf16 o [S][N]
    float* out_scales;     // MODE 0: scales of h [I / 128][S]
    long long b_expert_stride, sb_expert_stride;  // bytes / floats
    int K, N, S, n_tiles_n;
    // GATHER kernels (gate+up GEMM reading the caller's activations in place): A = x [T][K] e4m3,
    // SA = its scales [T][K / 128]; row `pos` of the sorted order is token sorted_slots[pos] / topk
    const int32_t* sorted_slots;
    int topk, T;
};

// Rows of a work item: 160, the most that leaves room for three LDS stages. An expert with up to 320
// rows then takes two passes over its weights (with 256 +- 16 rows per expert, the DeepSeek-V3 shape at
// 8192 tokens, 128-row items needed a third pass for half of the experts).
constexpr int kF8BM = 160;
constexpr int kF8ATile = kF8BM * 128;              // 20 KiB
constexpr int kF8BTile = 256 * 128;                // 32 KiB
constexpr int kF8Stage = kF8ATile + kF8BTile;      // 52 KiB
constexpr int kF8ScaleBase = 3 * kF8Stage;         // A scales: 3 stages x kF8BM floats
constexpr int kF8Lds = kF8ScaleBase + 3 * kF8BM * 4;   // 157.9 KiB
// (the gate+up epilogue's exchange buffer, kF8BM x 4 floats, lies in the stage the K loop used last)
static_assert(kF8Lds <= 160 * 1024 && kF8BM % 32 == 0 && kF8BM > 128 && kF8BM <= 192, "see the A-tile loads");

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
    uint32_t gvoff_a[(kF8BM + 63) / 64], gvoff_sa;  // GATHER: per-lane source offsets of the item's activation rows / scales
};

// GATHER (MODE 0 only): the activation tile's rows are fetched from the caller's x by token index
// (one 128-byte line per row and K-step either way), which saves writing and re-reading a
// permuted copy of x (k times its size).
template <int MODE, bool GATHER>
__global__ __launch_bounds__(512) void moe_fp8blk_gemm_kernel(const MoeFp8Params p) {
    static_assert(!GATHER || MODE == 0, "only the gate+up GEMM reads the caller's activations");
    // The A tile is loaded in NA = 3 pieces of 64 rows (8 per wave); of the third piece only rows 128..159
    // exist: waves 4..7 fetch what waves 0..3 fetch (same bytes to the same place), which keeps the number
    // of loads per wave uniform for the counted waits.
    constexpr int NW = 8, MT = kF8BM / 32, NT = 4, NA = (kF8BM + 63) / 64, SR = kF8BM / 8;
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
    const v4i srd_a = make_srd(p.A, GATHER ? (uint32_t)p.T * (uint32_t)p.K : (uint32_t)nk * (uint32_t)p.S * 128u);
    const v4i srd_sa = make_srd(p.SA, GATHER ? (uint32_t)p.T * (uint32_t)nk * 4u : (uint32_t)nk * (uint32_t)p.S * 4u);
    const uint32_t chunk16 = swz_chunk(8 * w + (lane >> 3), lane & 7);   // depends on w & 1 only
    // tile row this lane loads in piece i of the A tile
    auto piece_row = [&](int i) { return i < 2 ? 8 * (i * NW + w) + (lane >> 3) : 128 + 8 * (w & 3) + (lane >> 3); };
    auto piece_row0 = [&](int i) { return i < 2 ? 8 * (i * NW + w) : 128 + 8 * (w & 3); };

    // GATHER: sorted slot indices of the activation rows this lane loads for an item (NA tile pieces
    // and the scale row). They are fetched two items ahead with loads the compiler does not see
    // (a visible load would make it drain the whole load pipeline with vmcnt(0) before the
    // first use); the K loop's own waits cover them: they are queued behind the loads of the
    // item's first two K-steps and complete before the second wait returns.
    struct SlotIds { uint32_t a[NA]; uint32_t s; };
    auto issue_ids = [&](int idx, SlotIds& o) __attribute__((always_inline)) {
        if (idx >= it_end) idx = it_end - 1;
        const int row_start = scalar_load_x4(p.items + idx).y;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t off = (uint32_t)min(row_start + piece_row(i), p.S - 1) * 4u;
            asm volatile("global_load_dword %0, %1, %2" : "=v"(o.a[i]) : "v"(off), "s"(p.sorted_slots) : "memory");
        }
        const uint32_t off = (uint32_t)min(row_start + w * SR + min(lane, SR - 1), p.S - 1) * 4u;
        asm volatile("global_load_dword %0, %1, %2" : "=v"(o.s) : "v"(off), "s"(p.sorted_slots) : "memory");
    };
    auto landed_ids = [&](SlotIds& o) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NA; ++i) asm volatile("" : "+v"(o.a[i]));
        asm volatile("" : "+v"(o.s));
    };
    auto make_addr = [&](int idx, MoeFp8Addr& a, const SlotIds& ids) __attribute__((always_inline)) {
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
        if (GATHER) {
            // rows past the item's count are not fetched at all (bit 31: out of range, LDS gets zeros)
#pragma unroll
            for (int i = 0; i < NA; ++i)
                a.gvoff_a[i] = piece_row(i) < a.rows
                                   ? (ids.a[i] / (uint32_t)p.topk) * (uint32_t)p.K + chunk16 * 16u
                                   : 0x80000000u;
            a.gvoff_sa = w * SR + min(lane, SR - 1) < a.rows
                             ? (ids.s / (uint32_t)p.topk) * (uint32_t)nk * 4u
                             : 0x80000000u;
        }
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
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kF8ScaleBase + (uint32_t)w * SR * 4u);
    // LDS offset of this wave's part of A piece i within a stage
    const uint32_t lds_a2 = to_sgpr(lds0 + (uint32_t)(2 * NW + (w & 3)) * 1024u);
    auto a_piece_dst = [&](int stage, int i) {
        return (i < 2 ? lds_wave + (uint32_t)i * NW * 1024 : lds_a2) + (uint32_t)stage * kF8Stage;
    };
    uint32_t voff_a[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) voff_a[i] = (uint32_t)piece_row(i) * 128u + chunk16 * 16u;
    const uint32_t voff_sa = (uint32_t)((w * SR + lane) * 4);
    constexpr uint64_t kSaMask = (1ull << SR) - 1ull;

    auto issue_tile = [&](const MoeFp8Addr& a, int stage, int kt) {
        v4i sa = srd_a, sb = a.srd_b, ssa = srd_sa;
        if (!a.valid || kt >= nk) { sa.z = 0; sb.z = 0; ssa.z = 0; }
        const uint32_t row_base = (uint32_t)kt * (uint32_t)p.S + (uint32_t)a.row_start;
        const uint32_t dst = lds_wave + (uint32_t)stage * kF8Stage;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            if (GATHER) {
                dma16(sa, a_piece_dst(stage, i), a.gvoff_a[i], (uint32_t)kt * 128u);
            } else {
                v4i sai = sa;   // the piece's 8 rows lie past the item's count: nothing is fetched
                if (piece_row0(i) >= a.rows) sai.z = 0;
                dma16(sai, a_piece_dst(stage, i), voff_a[i], row_base * 128u);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(sb, dst + kF8ATile + i * NW * 1024, a.voff_b[i], (uint32_t)kt * 128u);
        if (GATHER) dma4_lanes(ssa, lds_sa_wave + (uint32_t)stage * (kF8BM * 4), a.gvoff_sa, (uint32_t)kt * 4u, kSaMask);
        else dma4_lanes(ssa, lds_sa_wave + (uint32_t)stage * (kF8BM * 4), voff_sa, row_base * 4u, kSaMask);
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
        uint32_t sa_rd = sa_rd0 + (uint32_t)st * (kF8BM * 4);
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

    auto epilogue = [&](const MoeFp8Addr& a, int free_stage) {
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
            // every wave is done with the K loop's last stage: its A tile becomes the exchange buffer
            const uint32_t xch = lds0 + (uint32_t)free_stage * kF8Stage;
            __syncthreads();
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
    SlotIds ids_cur{}, ids_nxt{}, ids_nn{};
    if (GATHER) {
        issue_ids(it, ids_cur);
        issue_ids(it + it_stride, ids_nxt);
        wait_vmcnt<0>();
        landed_ids(ids_cur);
        landed_ids(ids_nxt);
    }
    make_addr(it, cur, ids_cur);
    issue_tile(cur, 0, 0);
    if (depth == 2) issue_tile(cur, 1, 1);
    for (;;) {
        make_addr(it + it_stride, nxt, ids_nxt);
        if (GATHER) issue_ids(it + 2 * it_stride, ids_nn);
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
        epilogue(cur, st == 0 ? 2 : st - 1);
        it += it_stride;
        if (it >= it_end) break;
        cur = nxt;
        if (GATHER) {   // (asm: the copy must stay behind the K loop's waits)
#pragma unroll
            for (int i = 0; i < NA; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(ids_nxt.a[i]) : "v"(ids_nn.a[i]));
            asm volatile("v_mov_b32 %0, %1" : "=v"(ids_nxt.s) : "v"(ids_nn.s));
        }
    }
    wait_vmcnt<0>();
}

template <int MODE, bool GATHER>
static int launch_fp8blk_gemm(const MoeFp8Params& p, int max_items, hipStream_t s) {
    auto kern = moe_fp8blk_gemm_kernel<MODE, GATHER>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kF8Lds, configured)) return HK_ERR_LAUNCH;
    const int grid = min(max_items, moe_num_compute_units());
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kF8Lds, s, p);
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
    const int max_tiles = (int)(S / kF8BM) + E;
    L.max_items1 = max_tiles * (I / 128);
    L.max_items2 = max_tiles * ((H + 255) / 256);
    L.items1 = take((size_t)L.max_items1 * sizeof(MoeItem));
    L.items2 = take((size_t)L.max_items2 * sizeof(MoeItem));
    L.nitems = take(8);
    L.xq = L.xs = off;   // (the gate+up GEMM gathers the caller's activations in place: no permuted copy)
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

extern "C" int hk_moe_fp8blk_experts_ex(const void* x_e4m3, const float* x_scales, const void* w13,
                                        const float* w13_scales, const void* w2, const float* w2_scales,
                                        const float* topk_w, const int32_t* sorted_slots,
                                        const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                        int T, int H, int I, int E, int k, const void* y_add_bf16_or_null,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    if (!x_e4m3 || !x_scales || !w13 || !w13_scales || !w2 || !w2_scales || !topk_w || !sorted_slots ||
        !expert_offsets || !slot_to_pos || !y_bf16)
        return HK_ERR_NULL_POINTER;
    int st = fp8blk_check(T, H, I, E, k);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    if (((uintptr_t)x_e4m3 | (uintptr_t)w13 | (uintptr_t)w2 | (uintptr_t)y_bf16 | (uintptr_t)workspace) & 15u)
        return HK_ERR_BAD_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    const int S = T * k;
    int32_t* nitems = (int32_t*)(ws + L.nitems);
    moe_launch_build_items(expert_offsets, E, kF8BM, I / 128, (MoeItem*)(ws + L.items1), (H + 255) / 256,
                           (MoeItem*)(ws + L.items2), nitems, s);

    MoeFp8Params p{};
    p.A = (const uint8_t*)x_e4m3; p.SA = x_scales; p.S = S;   // gathered by token index inside the kernel
    p.sorted_slots = sorted_slots; p.topk = k; p.T = T;
    p.B = (const uint8_t*)w13; p.SB = w13_scales;
    p.b_expert_stride = (long long)2 * I * H; p.sb_expert_stride = (long long)(2 * I / 128) * (H / 128);
    p.items = (const MoeItem*)(ws + L.items1); p.num_items = nitems;
    p.out0 = ws + L.hq; p.out_scales = (float*)(ws + L.hs);
    p.K = H; p.N = I; p.n_tiles_n = I / 128;
    st = launch_fp8blk_gemm<0, true>(p, L.max_items1, s);
    if (st != HK_OK) return st;

    MoeFp8Params q{};
    q.A = ws + L.hq; q.SA = (const float*)(ws + L.hs); q.S = S;
    q.B = (const uint8_t*)w2; q.SB = w2_scales;
    q.b_expert_stride = (long long)H * I; q.sb_expert_stride = (long long)(H / 128) * (I / 128);
    q.items = (const MoeItem*)(ws + L.items2); q.num_items = nitems + 1;
    q.out0 = ws + L.o; q.out_scales = nullptr;
    q.K = I; q.N = H; q.n_tiles_n = (H + 255) / 256;
    st = launch_fp8blk_gemm<1, false>(q, L.max_items2, s);
    if (st != HK_OK) return st;
    return hk_moe_unpermute_add(ws + L.o, topk_w, slot_to_pos, T, k, H, y_add_bf16_or_null, y_bf16, stream);
}

extern "C" int hk_moe_fp8blk_experts(const void* x_e4m3, const float* x_scales, const void* w13,
                                     const float* w13_scales, const void* w2, const float* w2_scales,
                                     const float* topk_w, const int32_t* sorted_slots, const int32_t* expert_offsets,
                                     const int32_t* slot_to_pos, void* y_bf16, int T, int H, int I, int E, int k,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    return hk_moe_fp8blk_experts_ex(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, topk_w, sorted_slots,
                                    expert_offsets, slot_to_pos, y_bf16, T, H, I, E, k, nullptr, workspace,
                                    workspace_bytes, stream);
}

extern "C" int hk_moe_fp8blk_forward_ex(const void* x_e4m3, const float* x_scales, const float* router_logits,
                                        const float* router_bias_or_null, int n_group, int topk_group,
                                        float routed_scale, const void* w13, const float* w13_scales,
                                        const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                                        int E, int k, const void* y_add_bf16_or_null, void* workspace,
                                        size_t workspace_bytes, void* stream) {
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
    return hk_moe_fp8blk_experts_ex(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, (const float*)(ws + L.w),
                                    (const int32_t*)(ws + L.sorted), (const int32_t*)(ws + L.offsets),
                                    (const int32_t*)(ws + L.inv), y_bf16, T, H, I, E, k, y_add_bf16_or_null,
                                    workspace, workspace_bytes, stream);
}

extern "C" int hk_moe_fp8blk_forward(const void* x_e4m3, const float* x_scales, const float* router_logits,
                                     const float* router_bias_or_null, int n_group, int topk_group,
                                     float routed_scale, const void* w13, const float* w13_scales, const void* w2,
                                     const float* w2_scales, void* y_bf16, int T, int H, int I, int E, int k,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    return hk_moe_fp8blk_forward_ex(x_e4m3, x_scales, router_logits, router_bias_or_null, n_group, topk_group,
                                    routed_scale, w13, w13_scales, w2, w2_scales, y_bf16, T, H, I, E, k, nullptr,
                                    workspace, workspace_bytes, stream);
}
