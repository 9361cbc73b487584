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
    // (s_nop 4: when the kernel spills scalar registers, the compiler restores the base address with
    // v_readlane_b32 directly in front of the statement, and a vector-memory instruction that reads a
    // scalar register within five wait states of a vector-ALU write may see its old value.)
    struct SlotIds { uint32_t a[NA]; uint32_t s; };
    auto issue_ids = [&](int idx, SlotIds& o) __attribute__((always_inline)) {
        if (idx >= it_end) idx = it_end - 1;
        const int row_start = scalar_load_x4(p.items + idx).y;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t off = (uint32_t)min(row_start + piece_row(i), p.S - 1) * 4u;
            asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(o.a[i]) : "v"(off), "s"(p.sorted_slots) : "memory");
        }
        const uint32_t off = (uint32_t)min(row_start + w * SR + min(lane, SR - 1), p.S - 1) * 4u;
        asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(o.s) : "v"(off), "s"(p.sorted_slots) : "memory");
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
                        h[m][4 * q + j] = silu_mul(gv, up[j]);
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

// ------------------------------------------------------- grouped GEMM, pre-shuffled weights
// The kernel above moves both operands through LDS with two K-steps in flight; it is bound by how
// fast tiles are delivered to the CU (latency x bytes in flight) and by LDS traffic. This one is
// built around more bytes in flight and fewer LDS bytes per MFMA:
//   * 4 waves, one per SIMD (512 registers each). Wave w owns weight rows [64 w, +64) of the 256-row
//     tile (four MFMA fragments) x all rows of the item (up to 160 = ten fragments): 160 accumulator
//     registers, 4 MFMAs per activation fragment read;
//   * weights never touch LDS: the pre-shuffled layout (moe_fp8blk_preshuffle_kernel) stores, for
//     every (expert, n-tile, K-step), each wave's four fragments as contiguous 1 KiB pieces in lane
//     order, and the wave loads them straight into accumulation registers (AGPRs, which the MFMA
//     reads as its weight operand) four K-steps ahead: a ring of five sets of 32 registers;
//   * the activation tile (20 KiB + row scales) goes through a ring of five LDS stages, filled four
//     K-steps ahead by direct global->LDS loads (gate+up: gathered from the caller's x by token);
//   * the fp32 block scales are applied as before: every K-step's MFMAs write fresh partial sums,
//     acc += partial * (x_scale[row] * w_scale), here with hand-placed instructions: the FMAs of an
//     MFMA follow two MFMAs later, the next fragment's LDS reads and the loads of position + 3 are
//     spread over the MFMA slots. One wave per SIMD issues one instruction per four cycles, which
//     with 16 FMAs per fragment is as much as the MFMA pipe takes: no instruction is spent on
//     branches in the main path: every K-step runs all ten fragments (rows past an item's count are
//     zeros in LDS and are never stored), because accumulators behind branches cost register copies.
// The stream of (item, K-step) positions runs across item boundaries. All vector-memory loads are
// inline asm and counted by hand: per position a wave issues 14 loads (5 activation pieces, the row
// scales, 8 weight pieces; GATHER: 6 more per item for the slot ids), loads return in order, and the
// wait for position p + 1 sits in step p behind the loads of position p + 3: vmcnt(2 x 14). (Four
// positions ahead on five stages measured the same.) An item takes nk4 positions, nk rounded up to
// a multiple of the four register sets: its last position then always falls on set 3 and the
// epilogue code exists once (with a copy per set the kernel is 139 KB of code and every epilogue
// runs from a cold instruction cache). Padding positions fetch nothing: their LDS tile, row scales
// and weight registers read as zeros and add nothing.
// Results are bit-identical to the kernel above (same MFMA, K order and scaling FMAs).
constexpr int kF8sMT = kF8BM / 16;                       // at most 10 row fragments per item
// Items of nine fragments (144 rows): every K-step then runs nine fragments instead of ten. The host picks them
// when they do not add a pass over the weights (moe_fp8blk_item_rows): at 256 +- 16 rows per expert (the
// DeepSeek-V3-like layer at 8192 tokens) two items of up to 144 rows cover all but one expert in fifty.
constexpr int kF8BMShort = 144;
constexpr int kF8sStages = 4;                           // LDS stages = weight register sets = positions per trip of the K loop
constexpr int kF8sStage = 21504;                         // 160 x 128 B, then 16 x 12 row scales, padded to a multiple of 256 B
constexpr int kF8sXch = kF8sStages * kF8sStage;          // epilogue exchange buffer: 160 x 4 floats
constexpr int kF8sLds = kF8sXch + kF8BM * 16;            // 86.5 KiB
constexpr int kF8sBTile = 256 * 128;                     // one (n-tile, K-step) block of the pre-shuffled weights
constexpr int kF8sLoads = 14;                            // loads per wave and position
static_assert(kF8sStage >= kF8ATile + 16 * 12 * 4 && kF8sStage % 256 == 0 && kF8sLds <= 160 * 1024, "LDS plan");
static_assert((kF8sStages - 2) * kF8sLoads < 64 && kF8sStages == 4 && kF8sMT == 10 && kF8BMShort == 144, "vmcnt range; the slot plan below is written for nine or ten fragments");

// The weight ring lives in fixed accumulation registers: fragment F = 4 * set + n of the ring in
// a[8 F .. 8 F + 7] (low / high K half in the first / last four). Naming them in the constraints keeps the two
// 16-byte loads of a fragment and the MFMA that reads all 32 bytes on the same registers without copies.
#define HK_F8S_BREGS(X) \
    X(0, "{a[0:3]}", "{a[4:7]}", "{a[0:7]}") \
    X(1, "{a[8:11]}", "{a[12:15]}", "{a[8:15]}") \
    X(2, "{a[16:19]}", "{a[20:23]}", "{a[16:23]}") \
    X(3, "{a[24:27]}", "{a[28:31]}", "{a[24:31]}") \
    X(4, "{a[32:35]}", "{a[36:39]}", "{a[32:39]}") \
    X(5, "{a[40:43]}", "{a[44:47]}", "{a[40:47]}") \
    X(6, "{a[48:51]}", "{a[52:55]}", "{a[48:55]}") \
    X(7, "{a[56:59]}", "{a[60:63]}", "{a[56:63]}") \
    X(8, "{a[64:67]}", "{a[68:71]}", "{a[64:71]}") \
    X(9, "{a[72:75]}", "{a[76:79]}", "{a[72:79]}") \
    X(10, "{a[80:83]}", "{a[84:87]}", "{a[80:87]}") \
    X(11, "{a[88:91]}", "{a[92:95]}", "{a[88:95]}") \
    X(12, "{a[96:99]}", "{a[100:103]}", "{a[96:103]}") \
    X(13, "{a[104:107]}", "{a[108:111]}", "{a[104:111]}") \
    X(14, "{a[112:115]}", "{a[116:119]}", "{a[112:119]}") \
    X(15, "{a[120:123]}", "{a[124:127]}", "{a[120:127]}") \
    X(16, "{a[128:131]}", "{a[132:135]}", "{a[128:135]}") \
    X(17, "{a[136:139]}", "{a[140:143]}", "{a[136:143]}") \
    X(18, "{a[144:147]}", "{a[148:151]}", "{a[144:151]}") \
    X(19, "{a[152:155]}", "{a[156:159]}", "{a[152:159]}")

struct F8Cursor { int it, kt, expert, row_start, rows, n_tile; bool valid; };

// NONTEMP: weight loads with the non-temporal hint, for layers whose experts' rows fit one work item
// (the weights are then read once; see moe_mxfp4_stream4_kernel). At the DeepSeek-V3-like shape
// (256 rows per expert = two items) the second item would fetch them from HBM again: 4.24 against 4.12 ms.
template <int MODE, bool GATHER, bool NONTEMP = false, int MT = kF8sMT>
__global__ __launch_bounds__(256) void moe_fp8blk_stream_kernel(const MoeFp8Params p) {
    static_assert(!GATHER || MODE == 0, "only the gate+up GEMM reads the caller's activations");
    static_assert(MT == kF8sMT || MT == kF8BMShort / 16, "row fragments of an item");
    constexpr int NT = 4, NA = 5;
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
    const int nk4 = (nk + kF8sStages - 1) / kF8sStages * kF8sStages;
    const v4i srd_a = make_srd(p.A, GATHER ? (uint32_t)p.T * (uint32_t)p.K : (uint32_t)nk * (uint32_t)p.S * 128u);
    const v4i srd_sa = make_srd(p.SA, GATHER ? (uint32_t)p.T * (uint32_t)nk * 4u : (uint32_t)nk * (uint32_t)p.S * 4u);
    // Activation tile: wave w fetches rows [40 w, +40) in five 1 KiB pieces of 8 rows; lane l lands in
    // row + l / 8, physical chunk l % 8 and so fetches logical chunk swz(row, l % 8).
    auto piece_row = [&](int i) { return 40 * w + 8 * i + (lane >> 3); };
    // Row scales of a stage: [row % 16][row / 16, padded to 12] floats, so that a lane's scale of fragment
    // m sits at a fixed offset from its base. Wave w fetches slots [48 w, +48) with lanes 0..47.
    const int sf = 48 * w + min(lane, 47);
    const int scale_row = (sf % 12) < MT ? 16 * (sf % 12) + sf / 12 : -1;   // -1: padding slot, nothing fetched
    constexpr uint64_t kSaMask = (1ull << 48) - 1ull;

    // ---- cursors over this workgroup's stream of (item, K-step) positions -----------------------
    auto load_item = [&](F8Cursor& c) __attribute__((always_inline)) {
        c.valid = c.it < it_end;
        const v4i item = scalar_load_x4(p.items + (c.valid ? c.it : it_end - 1));
        c.expert = item.x; c.row_start = item.y; c.rows = item.z; c.n_tile = item.w;
    };
    auto advance = [&](F8Cursor& c) __attribute__((always_inline)) {
        if (++c.kt == nk4) { c.kt = 0; c.it += it_stride; load_item(c); }
    };
    F8Cursor cc{it0, 0}, cn, cf;   // compute position, the one after it, fetch position (+3)
    load_item(cc);
    cn = cc; advance(cn);
    cf = cc;

    // ---- GATHER: slot ids of the rows this lane fetches, one item ahead of the fetch cursor --------
    // (s_nop 4: when the kernel spills scalar registers, the compiler restores the base address with
    // v_readlane_b32 directly in front of the statement, and a vector-memory instruction that reads a
    // scalar register within five wait states of a vector-ALU write may see its old value.)
    struct SlotIds { uint32_t a[NA]; uint32_t s; };
    auto issue_ids = [&](int idx, SlotIds& o) __attribute__((always_inline)) {
        if (idx >= it_end) idx = it_end - 1;
        const int row_start = scalar_load_x4(p.items + idx).y;
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t off = (uint32_t)min(row_start + piece_row(i), p.S - 1) * 4u;
            asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(o.a[i]) : "v"(off), "s"(p.sorted_slots) : "memory");
        }
        const uint32_t off = (uint32_t)min(row_start + max(scale_row, 0), p.S - 1) * 4u;
        asm volatile("s_nop 4\n\tglobal_load_dword %0, %1, %2" : "=v"(o.s) : "v"(off), "s"(p.sorted_slots) : "memory");
    };
    auto landed_ids = [&](SlotIds& o) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NA; ++i) asm volatile("" : "+v"(o.a[i]));
        asm volatile("" : "+v"(o.s));
    };
    SlotIds ids_next{};
    // per-lane source offsets of the fetch cursor's item (GATHER: by token; else fixed tile offsets)
    uint32_t a_voff[NA], sa_voff;
    auto make_offsets = [&](const F8Cursor& c, const SlotIds& ids) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NA; ++i) {
            const uint32_t ch = swz_chunk(piece_row(i), lane & 7) * 16u;
            // GATHER: rows past the item's count are not fetched at all (bit 31: out of range, LDS gets zeros)
            if (GATHER) a_voff[i] = piece_row(i) < c.rows ? (ids.a[i] / (uint32_t)p.topk) * (uint32_t)p.K + ch : 0x80000000u;
            else a_voff[i] = (uint32_t)piece_row(i) * 128u + ch;
        }
        if (GATHER) sa_voff = scale_row >= 0 && scale_row < c.rows ? (ids.s / (uint32_t)p.topk) * (uint32_t)nk * 4u : 0x80000000u;
        else sa_voff = scale_row >= 0 ? (uint32_t)scale_row * 4u : 0x80000000u;
    };
    // uniform state of the fetch position, refreshed by fetch_begin() once per step
    v4i f_srd_a, f_srd_sa, f_srd_b;
    uint32_t f_soff_a, f_soff_sa, f_soff_b;
    int f_pieces;   // (not GATHER) pieces of this wave that hold rows of the item; the others fetch nothing
    // the fetch item's weight tile: found when the cursor enters the item, inside the branch that loads
    // the item (written as a conditional assignment elsewhere the compiler computes it at every position)
    auto b_tile_of = [&](const F8Cursor& c) __attribute__((always_inline)) {
        return p.B + (size_t)c.expert * p.b_expert_stride + (size_t)c.n_tile * nk * kF8sBTile;
    };
    const uint8_t* f_b_base = b_tile_of(cf);
    auto fetch_begin = [&]() __attribute__((always_inline)) {
        f_srd_a = srd_a; f_srd_sa = srd_sa;
        const bool live = cf.valid && cf.kt < nk;   // not past the stream's end, not a padding position
        if (!live) { f_srd_a.z = 0; f_srd_sa.z = 0; }
        f_srd_b = make_srd(f_b_base, live ? (uint32_t)nk * kF8sBTile : 0u);
        const uint32_t row_base = (uint32_t)cf.kt * (uint32_t)p.S + (uint32_t)cf.row_start;
        f_soff_a = GATHER ? (uint32_t)cf.kt * 128u : row_base * 128u;
        f_soff_sa = GATHER ? (uint32_t)cf.kt * 4u : row_base * 4u;
        f_soff_b = (uint32_t)cf.kt * kF8sBTile + (uint32_t)w * 8192u;
        f_pieces = GATHER ? NA : (cf.rows - 40 * w + 7) >> 3;
    };
    auto fetch_advance = [&]() __attribute__((always_inline)) {
        if (++cf.kt == nk4) {
            cf.kt = 0; cf.it += it_stride; load_item(cf);
            f_b_base = b_tile_of(cf);
            if (GATHER) {
                // the ids were requested when the cursor entered the previous item, ahead of that
                // position's loads, which an earlier step has waited for unless the item was shorter
                // than the wait's reach
                if (nk4 < kF8sStages) wait_vmcnt<0>();
                landed_ids(ids_next);
                make_offsets(cf, ids_next);
                issue_ids(cf.it + it_stride, ids_next);
            }
        }
    };

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave_a = to_sgpr(lds0 + (uint32_t)w * 5120u);
    const uint32_t lds_wave_sa = to_sgpr(lds0 + kF8ATile + (uint32_t)w * 192u);
    const uint32_t voff_b = lane * 16;
    struct BFrag { v4i lo, hi; };
    BFrag bw[kF8sStages][NT];   // weight fragments of four positions, in AGPRs
    // Load L (0..13) of the fetch position into LDS stage / register set PF. Order: an activation
    // piece or the scales, then a weight piece, alternating.
    auto fetch_load = [&]<int PF, int L>() __attribute__((always_inline)) {
        constexpr int kind = L < 12 ? (L & 1) : 1;            // 0: activation side, 1: weight piece
        constexpr int ai = L >> 1;                            // activation piece 0..4, 5 = row scales
        constexpr int bi = L < 12 ? (L >> 1) : L - 6;         // weight piece 0..7 = (fragment, K half)
        if constexpr (kind == 0 && ai < NA) {
            v4i s = f_srd_a;
            if (!GATHER && ai >= f_pieces) s.z = 0;
            dma16(s, lds_wave_a + PF * kF8sStage + ai * 1024, a_voff[ai], f_soff_a);
        } else if constexpr (kind == 0) {
            dma4_lanes(f_srd_sa, lds_wave_sa + PF * kF8sStage, sa_voff, f_soff_sa, kSaMask);
        } else {
            constexpr int n = bi >> 1, half = bi & 1, F = PF * NT + n;
            constexpr int imm = (n & 1) * 2048 + half * 1024;
            const uint32_t soff = f_soff_b + (n >= 2 ? 4096u : 0u);
            v4i& dst = half ? bw[PF][n].hi : bw[PF][n].lo;
#define HK_X(F_, LO, HI, ALL)                                                                                        \
    if constexpr (F == F_ && half == 0 && !NONTEMP)                                                                       \
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" : "=" LO(dst) : "v"(voff_b), "s"(f_srd_b), "s"(soff), "n"(imm) : "memory"); \
    if constexpr (F == F_ && half == 1 && !NONTEMP)                                                                       \
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" : "=" HI(dst) : "v"(voff_b), "s"(f_srd_b), "s"(soff), "n"(imm) : "memory"); \
    if constexpr (F == F_ && half == 0 && NONTEMP)                                                                        \
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4 nt" : "=" LO(dst) : "v"(voff_b), "s"(f_srd_b), "s"(soff), "n"(imm) : "memory"); \
    if constexpr (F == F_ && half == 1 && NONTEMP)                                                                        \
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4 nt" : "=" HI(dst) : "v"(voff_b), "s"(f_srd_b), "s"(soff), "n"(imm) : "memory");
            HK_F8S_BREGS(HK_X)
#undef HK_X
        }
    };
    auto fetch_all = [&]<int PF>() __attribute__((always_inline)) {
        fetch_load.template operator()<PF, 0>(); fetch_load.template operator()<PF, 1>();
        fetch_load.template operator()<PF, 2>(); fetch_load.template operator()<PF, 3>();
        fetch_load.template operator()<PF, 4>(); fetch_load.template operator()<PF, 5>();
        fetch_load.template operator()<PF, 6>(); fetch_load.template operator()<PF, 7>();
        fetch_load.template operator()<PF, 8>(); fetch_load.template operator()<PF, 9>();
        fetch_load.template operator()<PF, 10>(); fetch_load.template operator()<PF, 11>();
        fetch_load.template operator()<PF, 12>(); fetch_load.template operator()<PF, 13>();
    };
    auto landed = [&]<int PS>() __attribute__((always_inline)) {
#define HK_X(F_, LO, HI, ALL) \
    if constexpr (F_ / NT == PS) asm volatile("" : "+" LO(bw[PS][F_ % NT].lo), "+" HI(bw[PS][F_ % NT].hi));
        HK_F8S_BREGS(HK_X)
#undef HK_X
    };

    // ---- LDS -> registers -------------------------------------------------------------------------
    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = lds0 + r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = lds0 + r * 128u + swz_chunk(r, g + 4) * 16u;
    const uint32_t rd_sa = lds0 + kF8ATile + r * 48u;

    float acc[MT][NT][4];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[m][n][e] = 0.f;
    };
    v4f part[4] = {};        // partial sums of the last four MFMAs (slot n of a fragment writes part[n])
    v8i af[2];               // activation fragments, by fragment parity
    float xs_r[2];           // their rows' scales
    float sc[2][2] = {};     // by fragment parity: x_scale * w_scale of the gate (even) / up (odd) weight fragments
    float ws0 = 0.f, ws1 = 0.f;           // weight scales of the compute position
    float ws0_next = 0.f, ws1_next = 0.f; // ... of the position after it, requested one step earlier
    // D(16 weight rows x 16 rows) = W . A^T into fresh registers; weights from AGPRs
    auto mfma = [&]<int F>(v4f& d, const v8i& a) __attribute__((always_inline)) {
        const BFrag& b = bw[F / NT][F % NT];
        const v8i b8 = __builtin_shufflevector(b.lo, b.hi, 0, 1, 2, 3, 4, 5, 6, 7);
#define HK_X(F_, LO, HI, ALL) \
    if constexpr (F == F_) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=v"(d) : ALL(b8), "v"(a));
        HK_F8S_BREGS(HK_X)
#undef HK_X
    };
    // acc += part * s; placed by hand two MFMAs behind the one that produced `part` (the compiler does not
    // know the MFMA's latency), hence asm
    auto fma4 = [&](float (&a)[4], const v4f& pt, float s) __attribute__((always_inline)) {
        asm volatile("v_fma_f32 %0, %4, %8, %0\n\tv_fma_f32 %1, %5, %8, %1\n\tv_fma_f32 %2, %6, %8, %2\n\tv_fma_f32 %3, %7, %8, %3"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3])
                     : "v"(pt.x), "v"(pt.y), "v"(pt.z), "v"(pt.w), "v"(s));
    };
    // weight scales of a position, through the scalar cache, not waited for here
    // The scale rows of an item's two row blocks are found when a cursor enters the item (ws_rows_of, called
    // inside the branch that loads the item); a position then adds 4 kt.
    const float* ws_row0 = nullptr;
    const float* ws_row1 = nullptr;
    auto ws_rows_of = [&](const F8Cursor& c) __attribute__((always_inline)) {
        const float* sb = p.SB + (size_t)c.expert * p.sb_expert_stride;
        if (MODE == 0) {
            ws_row0 = sb + (size_t)c.n_tile * nk;                      // gate rows of the tile
            ws_row1 = sb + (size_t)(p.N / 128 + c.n_tile) * nk;        // up rows
        } else {
            ws_row0 = sb + (size_t)min(2 * c.n_tile + (w >> 1), p.N / 128 - 1) * nk;
            ws_row1 = ws_row0;
        }
    };
    auto request_ws = [&](const F8Cursor& c) __attribute__((always_inline)) {
        const uint32_t off = (uint32_t)min(c.kt, nk - 1) * 4u;   // a padding position multiplies zeros by the last K-step's scale
        asm volatile("s_load_dword %0, %1, %2" : "=s"(ws0_next) : "s"(ws_row0), "s"(off) : "memory");
        asm volatile("s_load_dword %0, %1, %2" : "=s"(ws1_next) : "s"(ws_row1), "s"(off) : "memory");
    };

    // Stores go through buffer descriptors that end at the item's last row: rows of the last
    // fragments beyond it are dropped by the range check (no per-lane row test, no 64-bit address
    // arithmetic); lanes that do not store carry bit 31 in their offset.
    auto epilogue = [&](const F8Cursor& a) __attribute__((always_inline)) {
        if (MODE == 1) {
            // lane (r, g) holds, for row 16 m + r, the columns n0 + 64 w + 32 q + 8 g .. +8 (q = 0, 1)
            const uint32_t pitch = (uint32_t)p.N * 2u;
            const v4i srd = make_srd((uint8_t*)p.out0 + (size_t)a.row_start * pitch, (uint32_t)a.rows * pitch);
            const int wcol0 = a.n_tile * 256 + w * 64;   // N % 128 == 0: a group of 32 columns is valid as a whole
            const bool ok0 = wcol0 < p.N, ok1 = wcol0 + 32 < p.N;
            uint32_t voff = r * pitch + (uint32_t)(wcol0 + 8 * (int)g) * 2u;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
#pragma unroll
                for (int q = 0; q < NT / 2; ++q) {
                    const float (&x)[4] = acc[m][2 * q];
                    const float (&y)[4] = acc[m][2 * q + 1];
                    v4i o4;
                    o4.x = pack_bf16(x[0], x[1]); o4.y = pack_bf16(x[2], x[3]);
                    o4.z = pack_bf16(y[0], y[1]); o4.w = pack_bf16(y[2], y[3]);
                    if (q == 0 ? ok0 : ok1)
                        asm volatile("buffer_store_dwordx4 %0, %1, %2, 0 offen offset:%3\n\ts_nop 1"
                                     :: "v"(o4), "v"(voff), "s"(srd), "n"(q * 64) : "memory");
                }
                voff += 16u * pitch;
            }
        } else {
            // h = silu(gate) * up for this wave's 32 of the tile's 128 h columns; the tile's 128
            // columns are one 1 x 128 quantization block, so the row maxima of the four waves are
            // combined through LDS.
            const size_t row0 = (size_t)a.n_tile * p.S + (size_t)a.row_start;
            const v4i srd_h = make_srd((uint8_t*)p.out0 + row0 * 128, (uint32_t)a.rows * 128u);
            const v4i srd_s = make_srd(p.out_scales + row0, (uint32_t)a.rows * 4u);
            uint32_t voff_h = r * 128u + 32u * (uint32_t)w + 8u * g;
            uint32_t voff_s = w == 0 && g == 0 ? r * 4u : 0x80000000u;
            float h[MT][8];
            const uint32_t xch = lds0 + kF8sXch;
#pragma unroll
            for (int m = 0; m < MT; ++m) {
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int j = 0; j < 4; ++j) h[m][4 * q + j] = silu_mul(acc[m][2 * q][j], acc[m][2 * q + 1][j]);
                float amax = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[m][i]));
                // maximum over the four lanes (r, 0..3) of a row: rows of 16 lanes swapped in registers
                const uint32_t am = __float_as_uint(amax);
                const auto s16 = __builtin_amdgcn_permlane16_swap(am, am, false, false);
                const uint32_t m1 = __float_as_uint(fmaxf(__uint_as_float(s16[0]), __uint_as_float(s16[1])));
                const auto s32 = __builtin_amdgcn_permlane32_swap(m1, m1, false, false);
                amax = fmaxf(__uint_as_float(s32[0]), __uint_as_float(s32[1]));
                const int row = 16 * m + (int)r;
                if (g == 0) *(lds_f32_mut_t*)(uintptr_t)(xch + (row * 4 + w) * 4) = amax;
            }
            __syncthreads();
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const int row = 16 * m + (int)r;
                const v4f am = *(lds_v4f_t*)(uintptr_t)(xch + row * 16);
                const float s = e4m3_block_scale(fmaxf(fmaxf(am.x, am.y), fmaxf(am.z, am.w)));
                const v2i q8 = quant8_e4m3(h[m], s);
                asm volatile("buffer_store_dwordx2 %0, %1, %2, 0 offen" :: "v"(q8), "v"(voff_h), "s"(srd_h) : "memory");
                asm volatile("buffer_store_dword %0, %1, %2, 0 offen" :: "v"(s), "v"(voff_s), "s"(srd_s) : "memory");
                voff_h += 16u * 128u;
                voff_s += 16u * 4u;
            }
            __syncthreads();   // the exchange buffer is rewritten by the next item's epilogue
        }
    };

    // ---- prologue: positions 0..3 in flight, the first position's first fragment in registers -------
    SlotIds ids0{};
    if (GATHER) {
        issue_ids(it0, ids0);
        issue_ids(it0 + it_stride, ids_next);
        wait_vmcnt<0>();
        landed_ids(ids0);
    }
    make_offsets(cf, ids0);
    fetch_begin(); fetch_all.template operator()<0>(); fetch_advance();
    fetch_begin(); fetch_all.template operator()<1>(); fetch_advance();
    fetch_begin(); fetch_all.template operator()<2>(); fetch_advance();
    ws_rows_of(cc);   // cn is still in this item (an item has at least four positions)
    request_ws(cc);
    zero_acc();
    wait_vmcnt<(kF8sStages - 2) * kF8sLoads>();
    block_barrier();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    asm volatile("" : "+s"(ws0_next), "+s"(ws1_next));   // the requested scales are in their registers from here on
    ws0 = ws0_next; ws1 = ws1_next;
    request_ws(cn);
    af[0] = lds_frag(rd_lo, rd_hi, 0);
    xs_r[0] = *(lds_f32_t*)(uintptr_t)rd_sa;

    // One stream position on LDS stage / weight register set P (both = position % 4). Every position
    // runs all ten fragments (rows past the item's count are zeros in LDS and are never stored): a
    // fragment count that varies would put the accumulators behind branches.
    auto step = [&]<int P>() __attribute__((always_inline)) {
        constexpr int PF = (P + kF8sStages - 1) % kF8sStages, PN = (P + 1) % kF8sStages;
        // af / xs_r / sc are double buffers indexed by fragment parity. With an odd number of fragments the
        // first fragment of consecutive positions would meet the last one of the position before in the same
        // buffer, so odd positions start on buffer 1 (an item has a multiple of four positions).
        constexpr int PAR = (MT & 1) ? (P & 1) : 0, PAR_PREV = (MT & 1) ? (PAR ^ 1) : 0, PAR_NEXT = PAR_PREV;
        fetch_begin();
        landed.template operator()<P>();
        const uint32_t a_lo = rd_lo + P * kF8sStage, a_hi = rd_hi + P * kF8sStage, a_sa = rd_sa + P * kF8sStage;
        // Behind fragment 8's third MFMA, when every LDS read of this position has been issued: the next
        // position's tile is waited for, its first fragment and scale are read, its weight scales arrive.
        auto transition = [&]() __attribute__((always_inline)) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this position's last LDS reads and the scale request
            asm volatile("" : "+s"(ws0_next), "+s"(ws1_next));
            wait_vmcnt<(kF8sStages - 2) * kF8sLoads>();
            block_barrier();   // everyone's part of the next position's tile has landed; everyone has read this position's
            af[PAR_NEXT] = lds_frag(rd_lo + PN * kF8sStage, rd_hi + PN * kF8sStage, 0);
            xs_r[PAR_NEXT] = *(lds_f32_t*)(uintptr_t)(rd_sa + PN * kF8sStage);
        };
        // Fragment M: four MFMA slots; the FMAs of an MFMA follow two slots later (fragment 0 starts with
        // those of fragment 9 of the previous K-step).
        auto block = [&]<int M>() __attribute__((always_inline)) {
            constexpr int MP = M == 0 ? MT - 1 : M - 1;   // the fragment whose last two FMA groups are still owed
            constexpr int B = (M + PAR) & 1, BN = B ^ 1;  // this fragment's buffer, the next one's
            constexpr int BP = M == 0 ? (MT - 1 + PAR_PREV) & 1 : BN;   // the buffer of fragment MP
            const v8i& a_cur = af[B];
            // slot 0
            mfma.template operator()<P * NT + 0>(part[0], a_cur);
            if constexpr (M < MT - 2) {
                af[BN] = lds_frag(a_lo, a_hi, (M + 1) * 2048);
                xs_r[BN] = *(lds_f32_t*)(uintptr_t)(a_sa + (M + 1) * 4);
            }
            fma4(acc[MP][2], part[2], sc[BP][0]);
            if constexpr (M <= 6) fetch_load.template operator()<PF, 2 * M>();
            __builtin_amdgcn_sched_barrier(0);
            // slot 1
            mfma.template operator()<P * NT + 1>(part[1], a_cur);
            fma4(acc[MP][3], part[3], sc[BP][1]);
            sc[B][0] = xs_r[B] * ws0;
            sc[B][1] = xs_r[B] * ws1;
            if constexpr (M <= 6) fetch_load.template operator()<PF, 2 * M + 1>();
            __builtin_amdgcn_sched_barrier(0);
            // slot 2
            mfma.template operator()<P * NT + 2>(part[2], a_cur);
            fma4(acc[M][0], part[0], sc[B][0]);
            if constexpr (M == MT - 2) {
                // fragment 9 is read here, ahead of the barrier that frees this stage
                af[BN] = lds_frag(a_lo, a_hi, (M + 1) * 2048);
                xs_r[BN] = *(lds_f32_t*)(uintptr_t)(a_sa + (M + 1) * 4);
            }
            __builtin_amdgcn_sched_barrier(0);
            // slot 3
            mfma.template operator()<P * NT + 3>(part[3], a_cur);
            fma4(acc[M][1], part[1], sc[B][1]);
            __builtin_amdgcn_sched_barrier(0);
        };
        block.template operator()<0>();
        block.template operator()<1>();
        block.template operator()<2>();
        block.template operator()<3>();
        block.template operator()<4>();
        block.template operator()<5>();
        block.template operator()<6>();
        block.template operator()<7>();
        if constexpr (MT > 9) block.template operator()<8>();
        // the last fragment, with the transition to the next position behind its first MFMA: ws0 / ws1 keep
        // this position's values until the end of the step
        {
            constexpr int M = MT - 1, MP = M - 1;
            constexpr int B = (M + PAR) & 1, BP = B ^ 1;
            const v8i& a_cur = af[B];
            mfma.template operator()<P * NT + 0>(part[0], a_cur);
            fma4(acc[MP][2], part[2], sc[BP][0]);
            __builtin_amdgcn_sched_barrier(0);
            mfma.template operator()<P * NT + 1>(part[1], a_cur);
            fma4(acc[MP][3], part[3], sc[BP][1]);
            sc[B][0] = xs_r[B] * ws0;
            sc[B][1] = xs_r[B] * ws1;
            transition();
            __builtin_amdgcn_sched_barrier(0);
            mfma.template operator()<P * NT + 2>(part[2], a_cur);
            fma4(acc[M][0], part[0], sc[B][0]);
            __builtin_amdgcn_sched_barrier(0);
            mfma.template operator()<P * NT + 3>(part[3], a_cur);
            fma4(acc[M][1], part[1], sc[B][1]);
            __builtin_amdgcn_sched_barrier(0);
        }
        fetch_advance();
        if constexpr (P == kF8sStages - 1) {
            if (cc.valid && cc.kt == nk4 - 1) {
                // the item is complete: the two FMA groups still owed, then the epilogue
                mfma_drain();
                fma4(acc[MT - 1][2], part[2], sc[(MT - 1 + PAR) & 1][0]);
                fma4(acc[MT - 1][3], part[3], sc[(MT - 1 + PAR) & 1][1]);
                epilogue(cc);
                zero_acc();
                // what the next K-step adds for "the last fragment of the previous K-step"
                sc[(MT - 1 + PAR) & 1][0] = 0.f; sc[(MT - 1 + PAR) & 1][1] = 0.f;
            }
        }
        cc = cn;
        if (++cn.kt == nk4) { cn.kt = 0; cn.it += it_stride; load_item(cn); ws_rows_of(cn); }
        ws0 = ws0_next; ws1 = ws1_next;
        request_ws(cn);
    };
    while (cc.valid) {
        step.template operator()<0>();
        step.template operator()<1>();
        step.template operator()<2>();
        step.template operator()<3>();
    }
    wait_vmcnt<0>();   // nothing may still be writing LDS when the workgroup retires
}

// Pre-shuffle of FP8 expert weights for moe_fp8blk_stream_kernel (offline, once per checkpoint).
// One thread per 16 bytes of the output. mode 0: gate+up matrix [E, 2N, K] (N = I); mode 1: down
// matrix [E, N, K] (N = H). Output: [E][n-tile][K-step][column wave 4][fragment 4][K half 2][lane 64][16],
// lane l = (r, g) holding row 64 wn + 16 f + r of the tile (moe_b_row) and bytes 16 (g + 4 half) .. +16
// of the K-step.
__global__ __launch_bounds__(256) void moe_fp8blk_preshuffle_kernel(const uint8_t* __restrict__ w, int N, int K,
                                                                    int mode, int n_tiles, long long expert_stride,
                                                                    uint8_t* __restrict__ out) {
    const int nk = K >> 7;
    const long long chunk = (long long)blockIdx.x * 256 + threadIdx.x;   // 16-byte chunk within the expert
    const long long per_expert = (long long)n_tiles * nk * (kF8sBTile / 16);
    if (chunk >= per_expert) return;
    const int e = blockIdx.y;
    const int lane = (int)(chunk & 63), half = (int)((chunk >> 6) & 1), f = (int)((chunk >> 7) & 3), wn = (int)((chunk >> 9) & 3);
    const long long blk = chunk >> 11;
    const int kt = (int)(blk % nk), nt = (int)(blk / nk);
    const int R = 64 * wn + 16 * f + (lane & 15);
    const int row = moe_b_row(mode, R, nt, N);
    const v4i v = *(const v4i*)(w + (size_t)e * expert_stride + (size_t)row * K + (size_t)kt * 128 + 16 * ((lane >> 4) + 4 * half));
    *(v4i*)(out + ((size_t)e * per_expert + chunk) * 16) = v;
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

template <int MODE, bool GATHER, bool NT, int MT>
static int launch_fp8blk_stream_nt(const MoeFp8Params& p, int max_items, hipStream_t s) {
    auto kern = moe_fp8blk_stream_kernel<MODE, GATHER, NT, MT>;
    static DeviceOnce configured;
    if (!set_lds_limit_once((const void*)kern, kF8sLds, configured)) return HK_ERR_LAUNCH;
    const int grid = min(max_items, moe_num_compute_units());
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), kF8sLds, s, p);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// bm: rows per work item the item lists were built for (kF8BM or kF8BMShort)
template <int MODE, bool GATHER>
static int launch_fp8blk_stream(const MoeFp8Params& p, int max_items, hipStream_t s, bool nt, int bm) {
    constexpr int kShort = kF8BMShort / 16;
    if (bm == kF8BMShort)
        return nt ? launch_fp8blk_stream_nt<MODE, GATHER, true, kShort>(p, max_items, s)
                  : launch_fp8blk_stream_nt<MODE, GATHER, false, kShort>(p, max_items, s);
    return nt ? launch_fp8blk_stream_nt<MODE, GATHER, true, kF8sMT>(p, max_items, s)
              : launch_fp8blk_stream_nt<MODE, GATHER, false, kF8sMT>(p, max_items, s);
}

// Rows per work item of the streaming kernels for a layer of T * k slots over E experts: 144 unless
// that costs a pass over the weights that 160 would not (judged at mean + two standard deviations of
// an expert's rows under uniform routing).
static int moe_fp8blk_item_rows(int T, int k, int E) {
    const double mu = (double)T * k / E, hi = mu + 2.0 * __builtin_sqrt(mu);
    const long long n_short = (long long)((hi + kF8BMShort - 1) / kF8BMShort);
    const long long n_long = (long long)((hi + kF8BM - 1) / kF8BM);
    return n_short <= n_long ? kF8BMShort : kF8BM;
}

// n-tiles of 256 weight rows of the two GEMMs: gate+up (mode 0: 128 h columns = 128 gate + 128 up rows
// per tile) and down (mode 1).
static inline int fp8blk_n_tiles(int mode, int N) { return mode == 0 ? N / 128 : (int)(((long long)N + 255) / 256); }

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
    const int max_tiles = (int)(S / kF8BMShort) + E;   // whichever item size the layer runs with
    L.max_items1 = max_tiles * (I / 128);
    L.max_items2 = max_tiles * ((H + 255) / 256);
    L.items1 = take((size_t)L.max_items1 * sizeof(MoeItem));
    L.items2 = take((size_t)L.max_items2 * sizeof(MoeItem));
    L.nitems = take(8);
    // e4m3 copy of x and its 1 x 128 scales, used only by the bf16-input entry point (the gate+up GEMM
    // gathers activation rows by token index: there is no permuted copy)
    L.xq = take((size_t)T * H); L.xs = take((size_t)T * (H / 128) * 4);
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

// Every argument check of the expert MLP, made before the first launch of a call (the forward entry points run
// quantization, routing and sort in front of the expert GEMMs: a call that is going to be refused must not have
// started any of them). x_e4m3 / x_scales: the caller's, or where the bf16 entry point will put them.
static int fp8blk_validate(const void* x_e4m3, const void* x_scales, const void* w13, const void* w13_scales,
                           const void* w2, const void* w2_scales, const void* y_bf16, int T, int H, int I, int E,
                           int k, int weight_layout, const void* y_add, const void* workspace,
                           size_t workspace_bytes) {
    if (weight_layout < 0 || weight_layout > 1) return HK_ERR_UNSUPPORTED;
    if (!x_e4m3 || !x_scales || !w13 || !w13_scales || !w2 || !w2_scales || !y_bf16) return HK_ERR_NULL_POINTER;
    const int st = fp8blk_check(T, H, I, E, k);
    if (st != HK_OK) return st;
    if (!workspace || workspace_bytes < fp8_ws_layout(T, H, I, E, k).total) return HK_ERR_WORKSPACE;
    if (((uintptr_t)x_e4m3 | (uintptr_t)w13 | (uintptr_t)w2 | (uintptr_t)y_bf16 | (uintptr_t)workspace |
         (uintptr_t)y_add) & 15u)
        return HK_ERR_BAD_ALIGNMENT;
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

// (0 for a shape the entry points refuse)
extern "C" size_t hk_moe_fp8blk_workspace_bytes(int T, int H, int I, int E, int k) {
    if (fp8blk_check(T, H, I, E, k) != HK_OK) return 0;
    return fp8_ws_layout(T, H, I, E, k).total;
}

extern "C" int hk_moe_fp8blk_preshuffle_bytes(int E, int N, int K, int mode, size_t* w_bytes) {
    if (!w_bytes) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 128) != 0 || (N % 128) != 0 || mode < 0 || mode > 1) return HK_ERR_BAD_SHAPE;
    *w_bytes = (size_t)E * fp8blk_n_tiles(mode, N) * (K / 128) * kF8sBTile;
    return HK_OK;
}

extern "C" int hk_moe_fp8blk_preshuffle(const void* w, int E, int N, int K, int mode, void* out_w, void* stream) {
    if (!w || !out_w) return HK_ERR_NULL_POINTER;
    if (E <= 0 || N <= 0 || K <= 0 || (K % 128) != 0 || (N % 128) != 0 || mode < 0 || mode > 1) return HK_ERR_BAD_SHAPE;
    if (E > 65535 || (long long)2 * N * K >= (1ll << 32)) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)w | (uintptr_t)out_w) & 15u) return HK_ERR_BAD_ALIGNMENT;
    const int n_tiles = fp8blk_n_tiles(mode, N);
    const long long chunks = (long long)n_tiles * (K / 128) * (kF8sBTile / 16);
    const long long rows = mode == 0 ? 2ll * N : N;
    hipLaunchKernelGGL(moe_fp8blk_preshuffle_kernel, dim3((unsigned)((chunks + 255) / 256), E), dim3(256), 0,
                       (hipStream_t)stream, (const uint8_t*)w, N, K, mode, n_tiles, rows * K, (uint8_t*)out_w);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_fp8blk_experts_ex2(const void* x_e4m3, const float* x_scales, const void* w13,
                                         const float* w13_scales, const void* w2, const float* w2_scales,
                                         const float* topk_w, const int32_t* sorted_slots,
                                         const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                         int T, int H, int I, int E, int k, int weight_layout,
                                         const void* y_add_bf16_or_null, void* workspace, size_t workspace_bytes,
                                         void* stream) {
    if (!topk_w || !sorted_slots || !expert_offsets || !slot_to_pos) return HK_ERR_NULL_POINTER;
    int st = fp8blk_validate(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, y_bf16, T, H, I, E, k, weight_layout,
                             y_add_bf16_or_null, workspace, workspace_bytes);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    const int S = T * k;
    int32_t* nitems = (int32_t*)(ws + L.nitems);
    const int bm = weight_layout == 1 ? moe_fp8blk_item_rows(T, k, E) : kF8BM;
    moe_launch_build_items(expert_offsets, E, bm, I / 128, (MoeItem*)(ws + L.items1), (H + 255) / 256,
                           (MoeItem*)(ws + L.items2), nitems, s);
    // non-temporal weight loads while most experts' rows fit one work item (their weights are then read once)
    const bool nt = moe_rows_fit_one_item(T, k, E, bm);

    MoeFp8Params p{};
    p.A = (const uint8_t*)x_e4m3; p.SA = x_scales; p.S = S;   // gathered by token index inside the kernel
    p.sorted_slots = sorted_slots; p.topk = k; p.T = T;
    p.B = (const uint8_t*)w13; p.SB = w13_scales;
    p.b_expert_stride = (long long)2 * I * H; p.sb_expert_stride = (long long)(2 * I / 128) * (H / 128);
    p.items = (const MoeItem*)(ws + L.items1); p.num_items = nitems;
    p.out0 = ws + L.hq; p.out_scales = (float*)(ws + L.hs);
    p.K = H; p.N = I; p.n_tiles_n = I / 128;
    if (weight_layout == 1) {
        p.b_expert_stride = (long long)fp8blk_n_tiles(0, I) * (H / 128) * kF8sBTile;
        st = launch_fp8blk_stream<0, true>(p, L.max_items1, s, nt, bm);
    } else {
        st = launch_fp8blk_gemm<0, true>(p, L.max_items1, s);
    }
    if (st != HK_OK) return st;

    MoeFp8Params q{};
    q.A = ws + L.hq; q.SA = (const float*)(ws + L.hs); q.S = S;
    q.B = (const uint8_t*)w2; q.SB = w2_scales;
    q.b_expert_stride = (long long)H * I; q.sb_expert_stride = (long long)(H / 128) * (I / 128);
    q.items = (const MoeItem*)(ws + L.items2); q.num_items = nitems + 1;
    q.out0 = ws + L.o; q.out_scales = nullptr;
    q.K = I; q.N = H; q.n_tiles_n = (H + 255) / 256;
    if (weight_layout == 1) {
        q.b_expert_stride = (long long)fp8blk_n_tiles(1, H) * (I / 128) * kF8sBTile;
        st = launch_fp8blk_stream<1, false>(q, L.max_items2, s, nt, bm);
    } else {
        st = launch_fp8blk_gemm<1, false>(q, L.max_items2, s);
    }
    if (st != HK_OK) return st;
    return hk_moe_unpermute_add(ws + L.o, topk_w, slot_to_pos, T, k, H, y_add_bf16_or_null, y_bf16, stream);
}

extern "C" int hk_moe_fp8blk_experts_ex(const void* x_e4m3, const float* x_scales, const void* w13,
                                        const float* w13_scales, const void* w2, const float* w2_scales,
                                        const float* topk_w, const int32_t* sorted_slots,
                                        const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                        int T, int H, int I, int E, int k, const void* y_add_bf16_or_null,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    return hk_moe_fp8blk_experts_ex2(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, topk_w, sorted_slots,
                                     expert_offsets, slot_to_pos, y_bf16, T, H, I, E, k, 0, y_add_bf16_or_null,
                                     workspace, workspace_bytes, stream);
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

extern "C" int hk_moe_fp8blk_forward_ex2(const void* x_e4m3, const float* x_scales, const float* router_logits,
                                         const float* router_bias_or_null, int n_group, int topk_group,
                                         float routed_scale, const void* w13, const float* w13_scales,
                                         const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                                         int E, int k, int weight_layout, const void* y_add_bf16_or_null,
                                         void* workspace, size_t workspace_bytes, void* stream) {
    if (!router_logits) return HK_ERR_NULL_POINTER;
    int st = fp8blk_validate(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, y_bf16, T, H, I, E, k, weight_layout,
                             y_add_bf16_or_null, workspace, workspace_bytes);
    if (st != HK_OK) return st;
    st = moe_topk_grouped_sigmoid_check(T, E, k, n_group, topk_group);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    uint8_t* ws = (uint8_t*)workspace;
    st = hk_moe_topk_grouped_sigmoid(router_logits, router_bias_or_null, T, E, k, n_group, topk_group, routed_scale,
                                     (int32_t*)(ws + L.ids), (float*)(ws + L.w), stream);
    if (st != HK_OK) return st;
    st = hk_moe_sort((const int32_t*)(ws + L.ids), T, k, E, (int32_t*)(ws + L.sorted), (int32_t*)(ws + L.offsets),
                     (int32_t*)(ws + L.inv), ws + L.sort_ws, hk_moe_sort_workspace_bytes(T, k, E), stream);
    if (st != HK_OK) return st;
    return hk_moe_fp8blk_experts_ex2(x_e4m3, x_scales, w13, w13_scales, w2, w2_scales, (const float*)(ws + L.w),
                                     (const int32_t*)(ws + L.sorted), (const int32_t*)(ws + L.offsets),
                                     (const int32_t*)(ws + L.inv), y_bf16, T, H, I, E, k, weight_layout,
                                     y_add_bf16_or_null, workspace, workspace_bytes, stream);
}

extern "C" int hk_moe_fp8blk_forward_ex(const void* x_e4m3, const float* x_scales, const float* router_logits,
                                        const float* router_bias_or_null, int n_group, int topk_group,
                                        float routed_scale, const void* w13, const float* w13_scales,
                                        const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                                        int E, int k, const void* y_add_bf16_or_null, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    return hk_moe_fp8blk_forward_ex2(x_e4m3, x_scales, router_logits, router_bias_or_null, n_group, topk_group,
                                     routed_scale, w13, w13_scales, w2, w2_scales, y_bf16, T, H, I, E, k, 0,
                                     y_add_bf16_or_null, workspace, workspace_bytes, stream);
}

extern "C" int hk_moe_fp8blk_forward_bf16(const void* x_bf16, const float* router_logits,
                                          const float* router_bias_or_null, int n_group, int topk_group,
                                          float routed_scale, const void* w13, const float* w13_scales,
                                          const void* w2, const float* w2_scales, void* y_bf16, int T, int H, int I,
                                          int E, int k, int weight_layout, const void* y_add_bf16_or_null,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    if (!x_bf16 || !router_logits) return HK_ERR_NULL_POINTER;
    if ((uintptr_t)x_bf16 & 15u) return HK_ERR_BAD_ALIGNMENT;
    // (the quantized copy of x and its scales will lie in the workspace: any non-null pointer stands in for them)
    int st = fp8blk_validate(workspace, workspace, w13, w13_scales, w2, w2_scales, y_bf16, T, H, I, E, k, weight_layout,
                             y_add_bf16_or_null, workspace, workspace_bytes);
    if (st != HK_OK) return st;
    st = moe_topk_grouped_sigmoid_check(T, E, k, n_group, topk_group);
    if (st != HK_OK) return st;
    const Fp8Ws L = fp8_ws_layout(T, H, I, E, k);
    uint8_t* ws = (uint8_t*)workspace;
    // every token is quantized once (T rows), ahead of the gather that repeats it for its k experts
    st = hk_fp8_quantize_rows_1x128(x_bf16, T, H, ws + L.xq, (float*)(ws + L.xs), stream);
    if (st != HK_OK) return st;
    return hk_moe_fp8blk_forward_ex2(ws + L.xq, (const float*)(ws + L.xs), router_logits, router_bias_or_null,
                                     n_group, topk_group, routed_scale, w13, w13_scales, w2, w2_scales, y_bf16, T,
                                     H, I, E, k, weight_layout, y_add_bf16_or_null, workspace, workspace_bytes,
                                     stream);
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
