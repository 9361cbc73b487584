// GEMM kernel body for few rows of A against a long weight matrix (decode shapes), shared by the FP8, BF16 and
// MXFP4 GEMMs (a K-step is 128 bytes per operand row in all three; the MFMA differs, and MXFP4 adds its scales).
#pragma once
#include "gemm_tile.h"
#include "hk_host.h"
#include "../../include/hk355.h"

namespace hk {

// Few rows of A against a long weight matrix (M <= 16 R): the GEMM is then one pass over
// B at HBM speed. A workgroup of NW waves owns 16 NF rows of B (as many columns of C, all rows of A); wave w walks
// its share of the K-steps on its own, without workgroup barriers: it fetches the 16 NF x 128-byte piece of B
// and the 16 R x 128-byte piece of A of a K-step with direct global->LDS loads (a row's 128 bytes by eight
// neighbouring lanes: whole cache lines, which a fetch straight into MFMA operand registers, a row per lane,
// does not give) into a ring of D stages of LDS that belongs to the wave alone, D - 1 K-steps in flight,
// and multiplies the stage that has landed. Rows past M or N and the 16-byte pieces past K lie outside the
// descriptors and arrive as zeros. The NW partial sums then meet in LDS and are added in wave order, so the
// result does not depend on timing and no second launch or workspace is needed (what the split-K path of the
// tile kernels spends on them).
constexpr int kSkinnyMaxM = 64;
// The bytes at `off` and `off + 4` of a descriptor's range (zero where outside), each in bits [7:0] of its
// component; waits for them. The wait states in front cover a descriptor that the compiler restores from a
// spilled register right before the statement.
__device__ __forceinline__ v2i scale_bytes_direct(v4i srd, uint32_t off) {
    int lo, hi;
    asm volatile(
        "s_nop 4\n\t"
        "buffer_load_ubyte %0, %2, %3, 0 offen\n\t"
        "buffer_load_ubyte %1, %2, %3, 0 offen offset:4\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(lo), "=&v"(hi)
        : "v"(off), "s"(srd)
        : "memory");
    return v2i{lo, hi};
}
// MMA: the operand type's MFMA on one 16-row x 128-byte fragment pair, `MMA::mma(acc, b, a)`. K is the operands'
// row length in BYTES (a multiple of 16); smem: the workgroup's dynamic LDS, skinny_lds_bytes(R, NW, D, scaled).
// MMA::kScaled (MXFP4): every operand row also has e8m0 block scales, 8 bytes per K-step, in rows of sa_pitch /
// sb_pitch bytes of which `row_bytes` are scales (any pitch and alignment); `MMA::mma(acc, b, a, sb, sa)` takes,
// per fragment, the lane's scale bytes of the K-step's two halves in bits [7:0] of .x / .y. A wave fetches the
// scales as it fetches the operands: the 128 scale bytes of each of its rows that cover 16 K-steps form a tile of
// the same shape as a K-step's operand bytes, loaded into one of two slots behind the stages, one such tile ahead.
// What such a fetch brings in beyond a row's scales (the next rows' bytes, zeros past the operand's last row,
// which ends the descriptor) belongs to K blocks past K, whose operand bytes arrive as zeros.
struct SkinnyScales {
    const uint8_t* SA; const uint8_t* SB; int sa_pitch, sb_pitch, row_bytes;
};
template <typename MMA, int R, int NW, int D, int NF = 2, bool NT = false>
__device__ __forceinline__ void gemm_skinny_body(
    uint8_t* smem, const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, float alpha, SkinnyScales sc = SkinnyScales{nullptr, nullptr, 0, 0, 0}) {
    constexpr bool kScaled = MMA::kScaled;
    constexpr int kRowsB = 16 * NF;   // rows of B per workgroup
    constexpr int kWBytes = kRowsB * BK, kStage = kWBytes + 16 * R * BK, kRegion = (D + (kScaled ? 2 : 0)) * kStage;
    constexpr int LPT = 2 * NF + 2 * R;   // loads per K-step (and per tile of scales)
    static_assert(D >= 2 && (D - 1 + (kScaled ? 1 : 0)) * LPT < 64, "vmcnt range");
    static_assert(NF == 1 || NF == 2, "one or two fragments of B per workgroup");
    static_assert(NW * R * NF * 1024 <= NW * kRegion, "the partial sums reuse the stages");
    const int lane = lane_id(), w = wave_id();
    const uint32_t r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * kRowsB;
    const int rows_b = N - n0 < kRowsB ? N - n0 : kRowsB;
    const v4i srd_b = make_srd(B + (size_t)n0 * K, (uint32_t)rows_b * (uint32_t)K);
    const v4i srd_a = make_srd(A, (uint32_t)M * (uint32_t)K);
    const int nk = (K + BK - 1) / BK;
    const int s0 = (int)((long long)nk * w / NW), n = (int)((long long)nk * (w + 1) / NW) - s0;

    // load i of a tile covers its rows 8 i .. 8 i + 7: lane l fetches, for LDS position l & 7 of row
    // 8 i + l / 8, the 16-byte chunk that the swizzle puts there
    uint32_t voff[2], tail_or[2];   // even / odd i (the swizzle of row 8 i + y depends on i's parity only)
#pragma unroll
    for (int par = 0; par < 2; ++par) {
        const uint32_t row = 8u * par + (lane >> 3);
        const uint32_t c = swz_chunk(row, lane & 7);
        voff[par] = row * (uint32_t)K + c * 16u;
        tail_or[par] = (int)(c * 16u) >= K - (nk - 1) * BK ? 0x80000000u : 0u;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
    const uint32_t region = to_sgpr(lds0 + (uint32_t)w * kRegion);
    // Without block scales a wave walks its K-steps from a start that differs from workgroup to workgroup (and
    // wraps around): rows whose length is a multiple of the memory channels' interleave (16 KiB: K = 8192 in bf16)
    // would otherwise have every workgroup at the same offset into its rows at the same time, i.e. in the same few
    // channels (M = 16, N = 8192, 16 KiB rows: 4.2 TB/s against 5.7 with rows of 18 KiB). The order is fixed by
    // the workgroup's index, so the result still does not depend on timing. (With scales the K-steps stay in
    // order: the scale tiles are fetched one ahead of a monotonic walk.)
    const int rot = kScaled || n == 0 ? 0 : (int)((blockIdx.x * 5u) % (uint32_t)n);
    auto step_of = [&](int kt_local) {
        const int x = kt_local + rot;
        return s0 + (x >= n ? x - n : x);
    };
    auto issue = [&](int stage, int kt_local) {
        const int kt = step_of(kt_local);
        const uint32_t k0 = (uint32_t)kt * BK, dst = region + (uint32_t)stage * kStage;
        const bool last = kt == nk - 1;
#pragma unroll
        for (int i = 0; i < 2 * NF; ++i) {
            const uint32_t vo = (voff[i & 1] + (uint32_t)(i >> 1) * 16u * (uint32_t)K) | (last ? tail_or[i & 1] : 0u);
            if constexpr (NT) dma16_nt(srd_b, dst + i * 1024, vo, k0);
            else dma16(srd_b, dst + i * 1024, vo, k0);
        }
#pragma unroll
        for (int i = 0; i < 2 * R; ++i)
            dma16(srd_a, dst + kWBytes + i * 1024, (voff[i & 1] + (uint32_t)(i >> 1) * 16u * (uint32_t)K) | (last ? tail_or[i & 1] : 0u), k0);
    };
    // scales (kScaled): tile c holds bytes [128 c, 128 c + 128) of the rows' scales, i.e. K-steps 16 c .. 16 c + 15
    v4i srd_sb = {0, 0, 0, 0}, srd_sa = {0, 0, 0, 0};
    uint32_t voff_sb[2] = {0, 0}, voff_sa[2] = {0, 0};
    if constexpr (kScaled) {
        srd_sb = make_srd(sc.SB + (size_t)n0 * sc.sb_pitch, (uint32_t)(rows_b - 1) * (uint32_t)sc.sb_pitch + (uint32_t)sc.row_bytes);
        srd_sa = make_srd(sc.SA, (uint32_t)(M - 1) * (uint32_t)sc.sa_pitch + (uint32_t)sc.row_bytes);
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const uint32_t row = 8u * par + (lane >> 3);
            const uint32_t c = swz_chunk(row, lane & 7);
            voff_sb[par] = row * (uint32_t)sc.sb_pitch + c * 16u;
            voff_sa[par] = row * (uint32_t)sc.sa_pitch + c * 16u;
        }
    }
    auto issue_scales = [&](int c) {
        const uint32_t dst = region + (uint32_t)(D + (c & 1)) * kStage, off = (uint32_t)c * 128u;
#pragma unroll
        for (int i = 0; i < 2 * NF; ++i)
            dma16(srd_sb, dst + i * 1024, voff_sb[i & 1] + (uint32_t)(i >> 1) * 16u * (uint32_t)sc.sb_pitch, off);
#pragma unroll
        for (int i = 0; i < 2 * R; ++i)
            dma16(srd_sa, dst + kWBytes + i * 1024, voff_sa[i & 1] + (uint32_t)(i >> 1) * 16u * (uint32_t)sc.sa_pitch, off);
    };
    auto wait_stages = [&](int in_flight) {   // at most `in_flight` of the most recently issued K-steps still fly
        switch (in_flight) {
            case 0: wait_vmcnt<0>(); break;
            case 1: wait_vmcnt<LPT>(); break;
            case 2: wait_vmcnt<(D > 3 ? 2 : 1) * LPT>(); break;
            case 3: wait_vmcnt<(D > 4 ? 3 : 1) * LPT>(); break;
            case 4: wait_vmcnt<(D > 5 ? 4 : 1) * LPT>(); break;
            default: wait_vmcnt<(D > 6 ? 5 : 1) * LPT>(); break;
        }
    };
    static_assert(D <= 7, "wait_stages covers up to five K-steps in flight");

    const uint32_t rd_lo = region + r * 128u + swz_chunk(r, g) * 16u;
    const uint32_t rd_hi = region + r * 128u + swz_chunk(r, g + 4) * 16u;
    v4f acc[R][NF];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int f = 0; f < NF; ++f) acc[i][f] = v4f{0.f, 0.f, 0.f, 0.f};

    // the wave's first tile of scales goes out in front of its first K-step: it has landed when that K-step has
    // (loads complete in order)
    const int c_last = (s0 + n - 1) >> 4;
    if constexpr (kScaled)
        if (n > 0) issue_scales(s0 >> 4);
#pragma unroll
    for (int p = 0; p < D - 1; ++p)
        if (p < n) issue(p, p);
    int st = 0;
    for (int kt = 0; kt < n; ++kt) {
        // K-step kt has landed. The count leaves the loads of scale tiles out: one of those among the loads
        // behind K-step kt makes the wait stricter than needed, never weaker
        wait_stages(min(n - 1 - kt, D - 2));
        const int ks = step_of(kt);
        if constexpr (kScaled) {
            // entering a tile of scales: the next one goes out, 16 K-steps (or what is left of the first tile)
            // before its first use; its slot's last reader was the K-step before this one
            if ((kt == 0 || (ks & 15) == 0) && (ks >> 4) < c_last) issue_scales((ks >> 4) + 1);
        }
        // the stage of K-step kt - 1 is free: its reads were waited for before its MFMAs
        if (kt + D - 1 < n) issue(st == 0 ? D - 1 : st - 1, kt + D - 1);
        const uint32_t so = (uint32_t)st * kStage;
        v8i wf[NF];
#pragma unroll
        for (int f = 0; f < NF; ++f) wf[f] = lds_frag(rd_lo + so, rd_hi + so, f * 16 * BK);
        if constexpr (kScaled) {
            v2i ws[NF], as[R];
            if ((sc.row_bytes & 3) != 0 && ks == nk - 1) {
                // The range check of a descriptor works on dwords: the dword of a scale tile that reaches across
                // the end of the operand's last row arrives as zero, and with it the last row_bytes % 4 scales of
                // that row. They belong to the last K-step, whose scale bytes every lane therefore fetches itself,
                // a byte at a time (the wave's loads have all landed: this is its last K-step).
#pragma unroll
                for (int f = 0; f < NF; ++f)
                    ws[f] = scale_bytes_direct(srd_sb, (16u * f + r) * (uint32_t)sc.sb_pitch + (uint32_t)ks * 8u + g);
#pragma unroll
                for (int i = 0; i < R; ++i)
                    as[i] = scale_bytes_direct(srd_sa, (16u * i + r) * (uint32_t)sc.sa_pitch + (uint32_t)ks * 8u + g);
            } else {
                // the lane's scale bytes: row r of each fragment, the 8 bytes of K-step ks, byte g of each half's dword
                const uint32_t sbase = region + (uint32_t)(D + ((ks >> 4) & 1)) * kStage + r * 128u +
                                       swz_chunk(r, (uint32_t)(ks & 15) >> 1) * 16u + (uint32_t)(ks & 1) * 8u;
                const uint32_t sh = 8u * g;
#pragma unroll
                for (int f = 0; f < NF; ++f) {
                    ws[f] = *(lds_v2i_t*)(uintptr_t)(sbase + f * 16 * BK);
                    ws[f].x = (int)((uint32_t)ws[f].x >> sh); ws[f].y = (int)((uint32_t)ws[f].y >> sh);
                }
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    as[i] = *(lds_v2i_t*)(uintptr_t)(sbase + kWBytes + i * 16 * BK);
                    as[i].x = (int)((uint32_t)as[i].x >> sh); as[i].y = (int)((uint32_t)as[i].y >> sh);
                }
            }
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const v8i af = lds_frag(rd_lo + so, rd_hi + so, kWBytes + i * 16 * BK);
#pragma unroll
                for (int f = 0; f < NF; ++f) MMA::mma(acc[i][f], wf[f], af, ws[f], as[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const v8i af = lds_frag(rd_lo + so, rd_hi + so, kWBytes + i * 16 * BK);
#pragma unroll
                for (int f = 0; f < NF; ++f) MMA::mma(acc[i][f], wf[f], af);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this stage's reads are done before a later load may overwrite it
        st = st == D - 1 ? 0 : st + 1;
    }
    // every wave is done with its stages (its loads have landed, its reads are complete): the partial sums take
    // their place
    __syncthreads();
    v4f* red = (v4f*)smem;   // [NW][R][NF][64]
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int f = 0; f < NF; ++f) red[((w * R + i) * NF + f) * 64 + lane] = acc[i][f];
    __syncthreads();
    for (int t = threadIdx.x; t < R * NF * 64; t += 64 * NW) {
        const int l = t & 63;
        v4f sum = red[t];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) sum += red[ww * R * NF * 64 + t];
        sum *= alpha;
        const int i = t / (NF * 64), f = (t >> 6) % NF;
        const int row = 16 * i + (l & 15), col = n0 + 16 * f + 4 * (l >> 4);
        if (row < M) {
            uint16_t* out = C + (size_t)row * N + col;
            if ((N & 3) == 0 && col + 3 < N) {
                *(uint2*)out = uint2{pack_bf16(sum.x, sum.y), pack_bf16(sum.z, sum.w)};
            } else {
                const float v[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < N) out[e] = (uint16_t)(pack_bf16(v[e], 0.f) & 0xffffu);
            }
        }
    }
}

constexpr int skinny_lds_bytes(int R, int NW, int D, bool scaled = false, int NF = 2) {
    return NW * (D + (scaled ? 2 : 0)) * (16 * NF + 16 * R) * BK;
}

// Whether a GEMM entry point takes this kernel when the caller does not pin one. nk: K-steps; with_ws: the caller
// gave a split-K workspace. From sweeps on an MI355X (M = 16 / 32 / 64, N = 512 ... 65536, K = 512 ... 16384
// bytes per row, against the tile kernels with and without split-K, the calls rotating over more weight matrices
// than the memory-side cache holds): up to 32 rows it wins by 2 to 64 % while it has at most one workgroup of 32
// rows per CU (N <= 8192 on 256 CUs); beyond that, up to 16 rows, from 32 K-steps on (8 to 25 %; with a shorter K,
// or with 17 to 32 rows and a long K, the 64x64-tile kernel's many tiles win by up to 20 %); with 33 to 64 rows it
// wins up to one workgroup per CU, except against split-K on few workgroups with a very long K. The MXFP4 form
// (wgs_per_cu = 2) wins by 5 to 75 % against the scaled tile kernels, whose scale fetches weigh more on few rows:
// from 32 K-steps on, up to 32 rows at any N and up to 64 rows up to two workgroups per CU (N <= 16384).
static inline bool use_skinny(int M, int N, int nk, bool with_ws, int cus, int max_m = kSkinnyMaxM, int wgs_per_cu = 1) {
    if (M > max_m) return false;
    const long long wgs = (N + 31) / 32;
    const bool long_k = nk >= 32;
    if (M <= 32) return wgs <= cus || (long_k && (M <= 16 || wgs_per_cu > 1));
    if (wgs > cus && !(long_k && wgs <= (long long)wgs_per_cu * cus)) return false;
    return !(with_ws && wgs * 2 <= cus && nk >= 96);
}

// KERNEL<R, NW, D, NF, NT>: the format's __global__ instantiation of the body
#define HK_SKINNY_LAUNCH(KERNEL, R, NW, D, NF, NT)                                                             \
    do {                                                                                                       \
        auto kern = KERNEL<R, NW, D, NF, NT>;                                                                  \
        constexpr int lds_bytes = skinny_lds_bytes(R, NW, D, false, NF);                                       \
        static_assert(lds_bytes <= 160 * 1024, "LDS of one CU");                                               \
        static DeviceOnce configured;                                                                          \
        if (!set_lds_limit_once((const void*)kern, lds_bytes, configured)) return HK_ERR_LAUNCH;               \
        hipLaunchKernelGGL(kern, dim3((N + 16 * NF - 1) / (16 * NF)), dim3(64 * NW), lds_bytes, stream,        \
                           (const uint8_t*)A, (const uint8_t*)B, (uint16_t*)C, M, N, K, alpha);                \
        return hipGetLastError() == hipSuccess ? HK_OK : HK_ERR_LAUNCH;                                        \
    } while (0)
// What a launch of the skinny kernel picks besides R (the rows of A):
//  - waves x stages per row count: the fastest of the combinations measured on an MI355X (N, K from 1024 to
//    28672; eight waves with three stages, two with seven and others are within 15 % of these);
//  - NF, the rows of B per workgroup: 16 instead of 32 while 32 would leave half of the CUs or more without a
//    workgroup (N <= 4096 on 256 CUs): a CU can only have so many bytes in flight, so weights that stream from
//    HBM want every CU (M = 16, N = 4096, K = 14336: 19.6 -> 12.9 us; N = 5760, 180 workgroups of 32 rows: 7.1
//    against 7.6 us with 16);
//  - NT, the non-temporal hint on the loads of B, from 8 MB of B on. Measured with the calls rotating over more
//    weight matrices than the 256 MB memory-side cache holds, which is what a model's decode step does, the hint
//    gains 3 to 18 % (M = 16, N = K = 8192: 14.2 -> 12.0 us); a benchmark that multiplies by the same 64 MB again
//    and again finds them in that cache and loses it with the hint, which is why small matrices, which a small
//    model may really keep there, go without.
// K in bytes per row.
constexpr long long kSkinnyNtBytes = 8ll << 20;
#define HK_SKINNY_PICK(KERNEL, R, NW, D)                                                          \
    do {                                                                                          \
        if (nf1) {                                                                                \
            if (nt) HK_SKINNY_LAUNCH(KERNEL, R, NW, D, 1, true);                                  \
            HK_SKINNY_LAUNCH(KERNEL, R, NW, D, 1, false);                                         \
        }                                                                                         \
        if (nt) HK_SKINNY_LAUNCH(KERNEL, R, NW, D, 2, true);                                      \
        HK_SKINNY_LAUNCH(KERNEL, R, NW, D, 2, false);                                             \
    } while (0)
#define HK_SKINNY_DISPATCH(KERNEL)                                                                \
    const bool nf1 = 2ll * ((N + 31) / 32) <= moe_num_compute_units();                            \
    const bool nt = (long long)N * K >= kSkinnyNtBytes;                                           \
    if (M <= 16) HK_SKINNY_PICK(KERNEL, 1, 4, 4);                                                 \
    if (M <= 32) HK_SKINNY_PICK(KERNEL, 2, 4, 3);                                                 \
    HK_SKINNY_PICK(KERNEL, 4, 4, 3)
// with block scales two slots of scales stand beside the stages: four waves with three stages fill the LDS of a CU
// at R = 2, and R = 4 (up to 64 rows) has room for two waves with four stages
constexpr int kSkinnyMaxMScaled = 64;

}  // namespace hk
