// MXFP4 fused MoE for gfx950: activation quantization, grouped gate+up GEMM with SiLU-mul and
// MX re-quantization in the epilogue, grouped down GEMM, weighted un-permute.
//
// The reference has no MoE code (no counterpart to cite); the GEMM core follows the 4-wave
// interleaved FP8/MXFP4 kernels of this library (LDS-direct loads into swizzled 128-byte-row
// tiles, ds_read_b128 fragments, v_mfma_scale_f32_16x16x128_f8f6f4 with in-MFMA e8m0 scales).
//
// Grouped GEMM: a work item is (m-tile, n-tile) where an m-tile is up to 128 consecutive rows
// (sorted positions) of one expert; the m-tile list is built on the device from
// expert_offsets. Each workgroup (4 waves, one per SIMD) computes a 128 x 256 tile; every wave
// spans all 128 rows and owns 64 of the 256 weight rows, so that 16-row fragments beyond the
// tile's real row count are skipped by all waves alike. Weights dominate HBM traffic at MoE
// shapes (about 128 rows per expert), so the K loop runs a three-stage LDS ring: two K-steps
// of operands are always in flight.
#include "gemm_tile.h"
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
// e2m1 code of v * 2^-e: round to nearest, ties to the even code, saturating at 6.
__device__ __forceinline__ uint32_t e2m1_code(float v, int e) {
    const float a = fabsf(ldexpf(v, -e));
    uint32_t c = (a > 0.25f) + (a >= 0.75f) + (a > 1.25f) + (a >= 1.75f) + (a > 2.5f) + (a >= 3.5f) +
                 (a > 5.0f);
    if (a != a) c = 7;  // NaN saturates like the oracle
    return c | ((__float_as_uint(v) >> 31) << 3);
}
__device__ __forceinline__ uint32_t pack8_e2m1(const float (&v)[8], int e) {
    uint32_t out = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) out |= e2m1_code(v[i], e) << (4 * i);
    return out;
}

// x [rows, cols] bf16 -> packed e2m1 [rows, cols/2] + e8m0 scales [rows, scale_pitch] (columns
// >= cols/32 are filled with 127). One thread per 8 elements, 4 threads per MX block.
__global__ __launch_bounds__(256) void mxfp4_quantize_rows_kernel(const uint16_t* __restrict__ x, int rows,
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
    const int e = mx_block_exponent(amax);
    if (in) *(uint32_t*)(packed + (size_t)row * (cols / 2) + c8 * 4) = pack8_e2m1(v, e);
    if ((c8 & 3) == 0) scales[(size_t)row * scale_pitch + (c8 >> 2)] = (uint8_t)(e + 127);
}

// ------------------------------------------------------------------------------ tile list
// m-tiles of up to kMoeBM rows, experts in order. tile_info[3*i] = {expert, first row, rows}.
constexpr int kMoeBM = 128;

__global__ __launch_bounds__(64) void moe_build_tiles_kernel(const int32_t* __restrict__ expert_offsets,
                                                             int E, int32_t* __restrict__ tile_info,
                                                             int32_t* __restrict__ num_tiles) {
    if (threadIdx.x != 0) return;
    int n = 0;
    for (int e = 0; e < E; ++e) {
        const int lo = expert_offsets[e], hi = expert_offsets[e + 1];
        for (int r = lo; r < hi; r += kMoeBM) {
            tile_info[3 * n + 0] = e;
            tile_info[3 * n + 1] = r;
            tile_info[3 * n + 2] = min(kMoeBM, hi - r);
            ++n;
        }
    }
    *num_tiles = n;
}

// ---------------------------------------------------------------------------- grouped GEMM
struct MoeGemmParams {
    const uint8_t* A;        // activations, packed e2m1 rows
    const uint8_t* SA;       // their e8m0 scales
    const uint8_t* B;        // expert weights, packed e2m1 [E][rows_b][b_pitch]
    const uint8_t* SB;       // their scales [E][rows_b][sb_pitch]
    const int32_t* sorted_slots;  // MODE 0: row p of the sorted order reads token sorted_slots[p]/topk
    const int32_t* tile_info;
    const int32_t* num_tiles;
    void* out0;              // MODE 0: packed h [S][out_pitch]; MODE 1: bf16 o [S][N]
    uint8_t* out_scales;     // MODE 0: e8m0 scales of h [S][out_scale_pitch]
    long long b_expert_stride, sb_expert_stride;
    int a_pitch, sa_pitch, b_pitch, sb_pitch;
    int out_pitch, out_scale_pitch;
    int K;                   // contraction length in elements
    int N;                   // MODE 0: I (h columns; weight rows i and I+i); MODE 1: output columns
    int topk, n_tiles_n;
};

constexpr int kMoeATile = kMoeBM * 128;                 // 16 KiB
constexpr int kMoeBTile = 256 * 128;                    // 32 KiB
constexpr int kMoeStage = kMoeATile + kMoeBTile;        // 48 KiB
constexpr int kMoeStages = 3;
constexpr int kMoeScaleA = kMoeBM * 8, kMoeScaleB = 256 * 8;
constexpr int kMoeScaleStage = kMoeScaleA + kMoeScaleB; // 3 KiB
constexpr int kMoeScaleBase = kMoeStages * kMoeStage;
constexpr int kMoeLds = kMoeScaleBase + kMoeStages * kMoeScaleStage;  // 153 KiB
constexpr int kMoeDmaPerTile = 4 + 8 + 1 + 2;           // A, B, A scales, B scales per wave

template <int MODE>
__global__ __launch_bounds__(256) void moe_mxfp4_gemm_kernel(const MoeGemmParams p) {
    constexpr int MT = 8, NT = 4, AD = 3, PG = 4;
    extern __shared__ __attribute__((aligned(2048))) uint8_t smem[];
    const int lane = lane_id(), w = wave_id();
    const int m_tile = blockIdx.x / p.n_tiles_n, n_tile = blockIdx.x % p.n_tiles_n;
    if (m_tile >= *p.num_tiles) return;
    const int expert = to_sgpr(p.tile_info[3 * m_tile + 0]);
    const int row_start = to_sgpr(p.tile_info[3 * m_tile + 1]);
    const int rows = to_sgpr(p.tile_info[3 * m_tile + 2]);
    const int mt_act = (rows + 15) >> 4;
    const int n0 = n_tile * (MODE == 0 ? 128 : 256);  // first h column / output column of the tile

    const int Kb = p.K >> 1;                 // contraction bytes per row
    const int nk = (Kb + 127) >> 7;
    const int tail_bytes = Kb - (nk - 1) * 128;  // valid bytes of the last K-step (16..128)

    const uint8_t* b_base = p.B + (size_t)expert * p.b_expert_stride;
    const uint8_t* sb_base = p.SB + (size_t)expert * p.sb_expert_stride;
    const int rows_b = MODE == 0 ? 2 * p.N : p.N;
    const v4i srd_a = make_srd(p.A, 0x7fffffffu);
    const v4i srd_sa = make_srd(p.SA, 0x7fffffffu);
    const v4i srd_b = make_srd(b_base, (uint32_t)rows_b * (uint32_t)p.b_pitch);
    const v4i srd_sb = make_srd(sb_base, (uint32_t)rows_b * (uint32_t)p.sb_pitch);

    // Weight row held by LDS row R of the B tile.
    auto b_row = [&](int R) -> int {
        if (MODE == 1) return min(n0 + b_row_to_col(R), p.N - 1);
        const int wn = R >> 6, t = (R >> 4) & 3, r = R & 15;
        const int hcol = 32 * wn + 8 * (r >> 2) + 4 * (t >> 1) + (r & 3);
        return (t & 1) * p.N + min(n0 + hcol, p.N - 1);
    };
    // Activation row (byte offset base) held by LDS row R of the A tile.
    auto a_row = [&](int R) -> uint32_t {
        const int pos = row_start + min(R, rows - 1);
        if (MODE == 0) return (uint32_t)(p.sorted_slots[pos] / p.topk);
        return (uint32_t)pos;
    };

    const uint32_t chunk = swz_chunk(8 * w + (lane >> 3), lane & 7);  // same for every load index
    const bool tail_oob = (int)(chunk * 16) >= tail_bytes;
    uint32_t voff_a[4], voff_b[8], voff_sa, voff_sb[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) voff_a[i] = a_row(8 * (i * 4 + w) + (lane >> 3)) * (uint32_t)p.a_pitch + chunk * 16u;
#pragma unroll
    for (int i = 0; i < 8; ++i) voff_b[i] = (uint32_t)b_row(8 * (i * 4 + w) + (lane >> 3)) * (uint32_t)p.b_pitch + chunk * 16u;
    voff_sa = a_row(32 * w + (lane >> 1)) * (uint32_t)p.sa_pitch + (lane & 1) * 4u;
#pragma unroll
    for (int j = 0; j < 2; ++j) voff_sb[j] = (uint32_t)b_row(32 * (2 * w + j) + (lane >> 1)) * (uint32_t)p.sb_pitch + (lane & 1) * 4u;

    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t lds_wave = to_sgpr(lds0 + (uint32_t)w * 1024u);
    const uint32_t lds_sa_wave = to_sgpr(lds0 + kMoeScaleBase + (uint32_t)w * 256u);
    const uint32_t lds_sb_wave = to_sgpr(lds0 + kMoeScaleBase + kMoeScaleA + (uint32_t)w * 512u);

    // All 15 loads of K-step kt into `stage`. Past the end of K they are issued against
    // zero-sized buffers (no traffic) so that the outstanding-load count stays uniform.
    auto issue_tile = [&](int stage, int kt) {
        v4i sa = srd_a, sb = srd_b, ssa = srd_sa, ssb = srd_sb;
        if (kt >= nk) { sa.z = 0; sb.z = 0; ssa.z = 0; ssb.z = 0; }
        const bool last = (kt == nk - 1) && tail_oob;
        const uint32_t k0 = (uint32_t)kt * 128u;
        const uint32_t dst = lds_wave + (uint32_t)stage * kMoeStage;
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(sa, dst + i * 4096, last ? 0x80000000u : voff_a[i], k0);
#pragma unroll
        for (int i = 0; i < 8; ++i) dma16(sb, dst + kMoeATile + i * 4096, last ? 0x80000000u : voff_b[i], k0);
        dma4(ssa, lds_sa_wave + (uint32_t)stage * kMoeScaleStage, voff_sa, (uint32_t)kt * 8u);
#pragma unroll
        for (int j = 0; j < 2; ++j)
            dma4(ssb, lds_sb_wave + (uint32_t)stage * kMoeScaleStage + j * 256, voff_sb[j], (uint32_t)kt * 8u);
    };

    const uint32_t r = lane & 15, g = lane >> 4;
    const uint32_t rd_lo = r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = r * 128u + swz_chunk(r, g + 4) * 16u;
    uint32_t a_lo[3], a_hi[3], b_lo[3], b_hi[3];
#pragma unroll
    for (int st = 0; st < 3; ++st) {
        a_lo[st] = lds0 + st * kMoeStage + rd_lo;
        a_hi[st] = lds0 + st * kMoeStage + rd_hi;
        b_lo[st] = lds0 + st * kMoeStage + kMoeATile + w * (64 * 128) + rd_lo;
        b_hi[st] = lds0 + st * kMoeStage + kMoeATile + w * (64 * 128) + rd_hi;
    }
    uint32_t sa_rd = lds0 + kMoeScaleBase + r * 8u;
    uint32_t sb_rd = lds0 + kMoeScaleBase + kMoeScaleA + (w * 64 + r) * 8u;
    asm volatile("" : "+v"(sa_rd), "+v"(sb_rd));
    const uint32_t sh = 8u * g;
    auto rd_scale = [&](uint32_t base, int stage, int f) -> v2i {
        return *(lds_v2i_t*)(uintptr_t)(base + stage * kMoeScaleStage + f * 128);
    };
    auto shift_scale = [&](v2i& s) {
        s.x = (int)((uint32_t)s.x >> sh);
        s.y = (int)((uint32_t)s.y >> sh);
    };
    struct Frag4 { v4i lo, hi; };
    auto rd_frag = [&](uint32_t lo, uint32_t hi, int imm) -> Frag4 {
        Frag4 f;
        f.lo = *(lds_v4i_t*)(uintptr_t)(lo + imm);
        f.hi = *(lds_v4i_t*)(uintptr_t)(hi + imm);
        return f;
    };
    auto mfma = [&](v4f& acc, const v4i& x, const v4i& y, int sx, int sy) {
        asm volatile(
            "v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
            : "+a"(acc)
            : "v"(x), "v"(y), "v"(sx), "v"(sy));
    };

    v4f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = v4f{0.f, 0.f, 0.f, 0.f};
    Frag4 bf[2][NT], af[4];
    v2i bs[2][NT], as[4];

    // ---- prologue: three K-steps in flight, fragments of the first in registers ----------
    issue_tile(0, 0);
    issue_tile(1, 1);
    issue_tile(2, 2);
    wait_vmcnt<2 * kMoeDmaPerTile>();
    block_barrier();
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        bf[0][n] = rd_frag(b_lo[0], b_hi[0], n * 2048);
        bs[0][n] = rd_scale(sb_rd, 0, n);
    }
#pragma unroll
    for (int m = 0; m < AD; ++m) {
        af[m] = rd_frag(a_lo[0], a_hi[0], m * 2048);
        as[m] = rd_scale(sa_rd, 0, m);
    }
#pragma unroll
    for (int n = 0; n < NT; ++n) shift_scale(bs[0][n]);
    shift_scale(as[0]);

    // One K-step. ST = LDS stage of this step, Q = parity of the B-fragment register set.
    auto step = [&]<int ST, int Q>(int kt) {
        constexpr int NS = (ST + 1) % 3;  // stage of the next K-step
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < mt_act) {
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    mfma(acc[m][n], bf[Q][n].lo, af[m & 3].lo, bs[Q][n].x, as[m & 3].x);
                    if (n == 0 && m <= PG) {
                        af[(m + AD) & 3] = rd_frag(a_lo[ST], a_hi[ST], (m + AD) * 2048);
                        as[(m + AD) & 3] = rd_scale(sa_rd, ST, m + AD);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    mfma(acc[m][n], bf[Q][n].hi, af[m & 3].hi, bs[Q][n].y, as[m & 3].y);
                    if (n == 2) shift_scale(as[(m + 1) & 3]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // keep the rotation of A buffers in step with the full schedule
                if (m <= PG) {
                    af[(m + AD) & 3] = rd_frag(a_lo[ST], a_hi[ST], (m + AD) * 2048);
                    as[(m + AD) & 3] = rd_scale(sa_rd, ST, m + AD);
                }
                shift_scale(as[(m + 1) & 3]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG) {
                // all reads of stage ST are issued; wait for them and for the next K-step's
                // loads (the K-step after that may stay in flight), then refill stage ST
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                wait_vmcnt<kMoeDmaPerTile>();
                block_barrier();
                issue_tile(ST, kt + 3);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG + 1) {
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    bf[Q ^ 1][n] = rd_frag(b_lo[NS], b_hi[NS], n * 2048);
                    bs[Q ^ 1][n] = rd_scale(sb_rd, NS, n);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG + 2) {
                af[0] = rd_frag(a_lo[NS], a_hi[NS], 0);
                as[0] = rd_scale(sa_rd, NS, 0);
                af[1] = rd_frag(a_lo[NS], a_hi[NS], 2048);
                as[1] = rd_scale(sa_rd, NS, 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (m == PG + 3) {
                af[2] = rd_frag(a_lo[NS], a_hi[NS], 2 * 2048);
                as[2] = rd_scale(sa_rd, NS, 2);
#pragma unroll
                for (int n = 0; n < NT; ++n) shift_scale(bs[Q ^ 1][n]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // stage cycles with period 3, register parity with period 2 -> unroll by 6
    int kt = 0;
    for (; kt + 5 < nk; kt += 6) {
        step.template operator()<0, 0>(kt);
        step.template operator()<1, 1>(kt + 1);
        step.template operator()<2, 0>(kt + 2);
        step.template operator()<0, 1>(kt + 3);
        step.template operator()<1, 0>(kt + 4);
        step.template operator()<2, 1>(kt + 5);
    }
    if (kt < nk) { step.template operator()<0, 0>(kt); ++kt; }
    if (kt < nk) { step.template operator()<1, 1>(kt); ++kt; }
    if (kt < nk) { step.template operator()<2, 0>(kt); ++kt; }
    if (kt < nk) { step.template operator()<0, 1>(kt); ++kt; }
    if (kt < nk) { step.template operator()<1, 0>(kt); ++kt; }
    wait_vmcnt<0>();
    mfma_drain();

    // ---- epilogue -------------------------------------------------------------------------
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
                if (col + 8 > p.N) continue;  // N % 8 == 0
                const v4f x = acc[m][2 * q], y = acc[m][2 * q + 1];
                v4i o4;
                o4.x = pack_bf16(x.x, x.y); o4.y = pack_bf16(x.z, x.w);
                o4.z = pack_bf16(y.x, y.y); o4.w = pack_bf16(y.z, y.w);
                *(v4i*)(out + pos * p.N + col) = o4;
            }
        }
    } else {
        uint8_t* hq = (uint8_t*)p.out0;
        const int hcol0 = n0 + 32 * w;  // this wave's MX block of h
        const bool col_ok = hcol0 < p.N;
        const bool last_n = n_tile == p.n_tiles_n - 1;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int row = 16 * m + (int)r;
            float h[8];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const v4f gt = acc[m][2 * q], up = acc[m][2 * q + 1];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float gv = gt[j];
                    h[4 * q + j] = gv / (1.0f + __expf(-gv)) * up[j];
                }
            }
            float amax = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(h[i]));
            amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            const int e = mx_block_exponent(amax);
            if (row < rows && col_ok) {
                const size_t pos = (size_t)(row_start + row);
                *(uint32_t*)(hq + pos * p.out_pitch + (hcol0 >> 1) + 4 * g) = pack8_e2m1(h, e);
                if (g == 0) p.out_scales[pos * p.out_scale_pitch + (hcol0 >> 5)] = (uint8_t)(e + 127);
            }
            if (row < rows && last_n && w == 0 && g == 1) {
                // neutral scale bytes in the padding columns of this row
                const size_t pos = (size_t)(row_start + row);
                for (int c = p.N >> 5; c < p.out_scale_pitch; ++c) p.out_scales[pos * p.out_scale_pitch + c] = 127;
            }
        }
    }
}

// ------------------------------------------------------------------------------ un-permute
// y[t, :] = bf16( sum_j w[t, j] * o[slot_to_pos[t*k + j], :] ), fp32 accumulation in choice order.
__global__ __launch_bounds__(256) void moe_unpermute_kernel(const uint16_t* __restrict__ o,
                                                            const float* __restrict__ w,
                                                            const int32_t* __restrict__ slot_to_pos, int T,
                                                            int k, int H, uint16_t* __restrict__ y) {
    const int t = blockIdx.x;
    for (int c = threadIdx.x; c < H / 8; c += 256) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        for (int j = 0; j < k; ++j) {
            const int pos = slot_to_pos[(size_t)t * k + j];
            const float wj = w[(size_t)t * k + j];
            const v4i raw = *(const v4i*)(o + (size_t)pos * H + c * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += wj * __uint_as_float((uint32_t)raw[i] << 16);
                acc[2 * i + 1] += wj * __uint_as_float((uint32_t)raw[i] & 0xffff0000u);
            }
        }
        v4i out;
        out.x = pack_bf16(acc[0], acc[1]); out.y = pack_bf16(acc[2], acc[3]);
        out.z = pack_bf16(acc[4], acc[5]); out.w = pack_bf16(acc[6], acc[7]);
        *(v4i*)(y + (size_t)t * H + c * 8) = out;
    }
}

static int round_up(int x, int m) { return (x + m - 1) / m * m; }

template <int MODE>
static int launch_moe_gemm(const MoeGemmParams& p, int max_m_tiles, hipStream_t s) {
    auto kern = moe_mxfp4_gemm_kernel<MODE>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kMoeLds) !=
            hipSuccess)
            return HK_ERR_LAUNCH;
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(max_m_tiles * p.n_tiles_n), dim3(256), kMoeLds, s, p);
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
    hipLaunchKernelGGL(mxfp4_quantize_rows_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t*)x_bf16, rows, cols, (uint8_t*)packed,
                       (uint8_t*)scales, scale_pitch);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

extern "C" int hk_moe_unpermute(const void* o_bf16, const float* w, const int32_t* slot_to_pos, int T, int k,
                                int H, void* y_bf16, void* stream) {
    if (!o_bf16 || !w || !slot_to_pos || !y_bf16) return HK_ERR_NULL_POINTER;
    if (T <= 0 || k <= 0 || H <= 0 || (H % 8) != 0) return HK_ERR_BAD_SHAPE;
    if (((uintptr_t)o_bf16 | (uintptr_t)y_bf16) & 15u) return HK_ERR_BAD_ALIGNMENT;
    hipLaunchKernelGGL(moe_unpermute_kernel, dim3(T), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)o_bf16,
                       w, slot_to_pos, T, k, H, (uint16_t*)y_bf16);
    return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;
}

// Workspace layout of hk_moe_mxfp4_forward (all regions 256-byte aligned).
struct MoeWs {
    size_t ids, w, sorted, offsets, inv, sort_ws, tiles, ntiles, xq, xs, hq, hs, o, total;
};
static MoeWs moe_ws_layout(int T, int H, int I, int E, int k) {
    MoeWs L;
    size_t off = 0;
    auto take = [&](size_t bytes) { size_t at = off; off = (off + bytes + 255) / 256 * 256; return at; };
    const size_t S = (size_t)T * k;
    L.ids = take(S * 4); L.w = take(S * 4); L.sorted = take(S * 4); L.offsets = take((size_t)(E + 1) * 4);
    L.inv = take(S * 4); L.sort_ws = take(hk_moe_sort_workspace_bytes(T, k, E));
    const size_t max_tiles = S / kMoeBM + E;
    L.tiles = take(max_tiles * 12); L.ntiles = take(4);
    L.xq = take((size_t)T * (H / 2)); L.xs = take((size_t)T * round_up(H / 32, 8));
    L.hq = take(S * (I / 2)); L.hs = take(S * round_up(I / 32, 8));
    L.o = take(S * (size_t)H * 2);
    L.total = off;
    return L;
}

extern "C" size_t hk_moe_mxfp4_workspace_bytes(int T, int H, int I, int E, int k) {
    if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0) return 0;
    return moe_ws_layout(T, H, I, E, k).total;
}

static int moe_mxfp4_check(int T, int H, int I, int E, int k, int w13_scale_pitch, int w2_scale_pitch) {
    if (T <= 0 || E <= 0 || k <= 0 || k > E || k > 64 || E > 512) return HK_ERR_BAD_SHAPE;
    if (H <= 0 || I <= 0 || (H % 32) != 0 || (I % 32) != 0) return HK_ERR_BAD_SHAPE;
    if (w13_scale_pitch < H / 32 || (w13_scale_pitch % 8) != 0 || w2_scale_pitch < I / 32 ||
        (w2_scale_pitch % 8) != 0)
        return HK_ERR_BAD_SHAPE;
    if ((long long)T * k >= (1ll << 24) || (long long)T * k * (I / 2) >= (1ll << 31) ||
        (long long)T * (H / 2) >= (1ll << 31) || (long long)2 * I * (H / 2) >= (1ll << 31) ||
        (long long)H * (I / 2) >= (1ll << 31))
        return HK_ERR_BAD_SHAPE;
    return HK_OK;
}

// Expert MLP on already routed and sorted tokens (steps 3-6 of the forward pass).
extern "C" int hk_moe_mxfp4_experts(const void* x_bf16, const void* w13, const void* w13_scales,
                                    int w13_scale_pitch, const void* w2, const void* w2_scales,
                                    int w2_scale_pitch, const float* topk_w, const int32_t* sorted_slots,
                                    const int32_t* expert_offsets, const int32_t* slot_to_pos, void* y_bf16,
                                    int T, int H, int I, int E, int k, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    if (!x_bf16 || !w13 || !w13_scales || !w2 || !w2_scales || !topk_w || !sorted_slots || !expert_offsets ||
        !slot_to_pos || !y_bf16)
        return HK_ERR_NULL_POINTER;
    int st = moe_mxfp4_check(T, H, I, E, k, w13_scale_pitch, w2_scale_pitch);
    if (st != HK_OK) return st;
    const MoeWs L = moe_ws_layout(T, H, I, E, k);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    if (((uintptr_t)x_bf16 | (uintptr_t)w13 | (uintptr_t)w2 | (uintptr_t)y_bf16 | (uintptr_t)workspace) & 15u)
        return HK_ERR_BAD_ALIGNMENT;
    if (((uintptr_t)w13_scales | (uintptr_t)w2_scales) & 3u) return HK_ERR_BAD_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    uint8_t* ws = (uint8_t*)workspace;
    const int S = T * k;
    const int xs_pitch = round_up(H / 32, 8), hs_pitch = round_up(I / 32, 8);
    const int max_tiles = S / kMoeBM + E;

    st = hk_mxfp4_quantize_rows(x_bf16, T, H, ws + L.xq, ws + L.xs, xs_pitch, stream);
    if (st != HK_OK) return st;
    hipLaunchKernelGGL(moe_build_tiles_kernel, dim3(1), dim3(64), 0, s, expert_offsets, E,
                       (int32_t*)(ws + L.tiles), (int32_t*)(ws + L.ntiles));

    MoeGemmParams p{};
    p.A = ws + L.xq; p.SA = ws + L.xs; p.a_pitch = H / 2; p.sa_pitch = xs_pitch;
    p.B = (const uint8_t*)w13; p.SB = (const uint8_t*)w13_scales;
    p.b_pitch = H / 2; p.sb_pitch = w13_scale_pitch;
    p.b_expert_stride = (long long)2 * I * (H / 2); p.sb_expert_stride = (long long)2 * I * w13_scale_pitch;
    p.sorted_slots = sorted_slots; p.tile_info = (const int32_t*)(ws + L.tiles);
    p.num_tiles = (const int32_t*)(ws + L.ntiles);
    p.out0 = ws + L.hq; p.out_scales = ws + L.hs; p.out_pitch = I / 2; p.out_scale_pitch = hs_pitch;
    p.K = H; p.N = I; p.topk = k; p.n_tiles_n = (I + 127) / 128;
    st = launch_moe_gemm<0>(p, max_tiles, s);
    if (st != HK_OK) return st;

    MoeGemmParams q{};
    q.A = ws + L.hq; q.SA = ws + L.hs; q.a_pitch = I / 2; q.sa_pitch = hs_pitch;
    q.B = (const uint8_t*)w2; q.SB = (const uint8_t*)w2_scales;
    q.b_pitch = I / 2; q.sb_pitch = w2_scale_pitch;
    q.b_expert_stride = (long long)H * (I / 2); q.sb_expert_stride = (long long)H * w2_scale_pitch;
    q.sorted_slots = sorted_slots; q.tile_info = p.tile_info; q.num_tiles = p.num_tiles;
    q.out0 = ws + L.o; q.out_scales = nullptr; q.out_pitch = 0; q.out_scale_pitch = 0;
    q.K = I; q.N = H; q.topk = k; q.n_tiles_n = (H + 255) / 256;
    st = launch_moe_gemm<1>(q, max_tiles, s);
    if (st != HK_OK) return st;

    return hk_moe_unpermute(ws + L.o, topk_w, slot_to_pos, T, k, H, y_bf16, stream);
}

extern "C" int hk_moe_mxfp4_forward(const void* x_bf16, const float* router_logits, const void* w13,
                                    const void* w13_scales, int w13_scale_pitch, const void* w2,
                                    const void* w2_scales, int w2_scale_pitch, void* y_bf16, int T, int H, int I,
                                    int E, int k, void* workspace, size_t workspace_bytes, void* stream) {
    if (!router_logits) return HK_ERR_NULL_POINTER;
    int st = moe_mxfp4_check(T, H, I, E, k, w13_scale_pitch, w2_scale_pitch);
    if (st != HK_OK) return st;
    const MoeWs L = moe_ws_layout(T, H, I, E, k);
    if (!workspace || workspace_bytes < L.total) return HK_ERR_WORKSPACE;
    uint8_t* ws = (uint8_t*)workspace;
    st = hk_moe_topk_softmax(router_logits, T, E, k, (int32_t*)(ws + L.ids), (float*)(ws + L.w), stream);
    if (st != HK_OK) return st;
    st = hk_moe_sort((const int32_t*)(ws + L.ids), T, k, E, (int32_t*)(ws + L.sorted), (int32_t*)(ws + L.offsets),
                     (int32_t*)(ws + L.inv), ws + L.sort_ws, hk_moe_sort_workspace_bytes(T, k, E), stream);
    if (st != HK_OK) return st;
    return hk_moe_mxfp4_experts(x_bf16, w13, w13_scales, w13_scale_pitch, w2, w2_scales, w2_scale_pitch,
                                (const float*)(ws + L.w), (const int32_t*)(ws + L.sorted),
                                (const int32_t*)(ws + L.offsets), (const int32_t*)(ws + L.inv), y_bf16, T, H, I, E,
                                k, workspace, workspace_bytes, stream);
}
