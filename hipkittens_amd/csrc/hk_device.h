// Device-side building blocks shared by the gfx950 kernels: buffer descriptors,
// direct global->LDS loads, the LDS tile swizzle, MFMA wrappers, bf16 packing and
// the XCD-aware workgroup order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hk {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const v4i lds_v4i_t;
typedef __attribute__((address_space(3))) const v2i lds_v2i_t;

constexpr int kWave = 64;
constexpr int kNumXcd = 8;
constexpr int kCuPerXcd = 32;

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// Wave index as a scalar (SGPR) value.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }
__device__ __forceinline__ uint32_t to_sgpr(uint32_t x) { return __builtin_amdgcn_readfirstlane(x); }

// Raw (unstrided, unswizzled) buffer descriptor over [base, base+bytes).
// Plays the role of make_srsrc in the reference
// (include/ops/warp/memory/util/util.cuh:72-88).
__device__ __forceinline__ v4i make_srd(const void* base, uint32_t bytes) {
    uint64_t p = (uint64_t)base;
    v4i s;
    s.x = to_sgpr((uint32_t)p);
    s.y = to_sgpr((uint32_t)(p >> 32) & 0xffffu);
    s.z = to_sgpr(bytes);
    s.w = 0x00020000;
    return s;
}

// One `buffer_load_dwordx4 ... lds`: every lane fetches 16 bytes from
// srd.base + voff + soff and the wave's 1024 bytes land contiguously in LDS at
// lds_base + 16*lane. lds_base and soff must be wave-uniform.
// Written as inline asm so that the compiler's LDS-DMA alias tracking does not
// force vmcnt(0) in front of every later LDS read; completion is awaited
// explicitly with wait_vmcnt<N>().
__device__ __forceinline__ void dma16(v4i srd, uint32_t lds_base, uint32_t voff, uint32_t soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen lds"
        :
        : "s"(lds_base), "v"(voff), "s"(srd), "s"(soff)
        : "memory", "m0");
}

// dma16 with the non-temporal hint, for data that is read once (the weights of a decode GEMM): it need not
// displace what the caches hold for re-use.
__device__ __forceinline__ void dma16_nt(v4i srd, uint32_t lds_base, uint32_t voff, uint32_t soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen nt lds"
        :
        : "s"(lds_base), "v"(voff), "s"(srd), "s"(soff)
        : "memory", "m0");
}

// 4-byte direct global->LDS load (64 lanes -> 256 contiguous LDS bytes).
__device__ __forceinline__ void dma4(v4i srd, uint32_t lds_base, uint32_t voff, uint32_t soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dword %1, %2, %3 offen lds"
        :
        : "s"(lds_base), "v"(voff), "s"(srd), "s"(soff)
        : "memory", "m0");
}

// dma16 restricted to the lanes set in `mask` (lane l still lands at lds_base + 16*l).
__device__ __forceinline__ void dma16_lanes(v4i srd, uint32_t lds_base, uint32_t voff, uint32_t soff,
                                            uint64_t mask) {
    uint64_t saved;
    asm volatile(
        "s_mov_b64 %0, exec\n\t"
        "s_mov_b64 exec, %5\n\t"
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %2, %3, %4 offen lds\n\t"
        "s_mov_b64 exec, %0"
        : "=&s"(saved)
        : "s"(lds_base), "v"(voff), "s"(srd), "s"(soff), "s"(mask)
        : "memory", "m0");
}

// dma4 restricted to the lanes set in `mask` (lane l still lands at lds_base + 4*l).
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

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Fixes the position of everything around it: memory operations may not be moved across the
// empty asm (compiler fence) and the machine scheduler may not move anything across the
// scheduling barrier. Used between the slots of the hand-interleaved schedules.
__device__ __forceinline__ void slot_fence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void block_barrier() { __builtin_amdgcn_s_barrier(); }

// LDS tile layout for K-contiguous operand tiles with 128-byte rows: the 16-byte
// chunk index is XORed with bits [1..3] of the row. With lane l of an MFMA
// operand read touching row l%16 and chunk l/16 this is free of bank conflicts
// for ds_read_b128 (formula as in kernels/gemm/fp8fp32/FP8_4wave/utils.cpp:123-128).
__device__ __forceinline__ uint32_t swz_chunk(uint32_t row, uint32_t chunk) {
    return chunk ^ ((row >> 1) & 7u);
}

// 16x128 (fp8) / 16x256 (fp4) MFMA operand fragment: lane l holds row l%16 and the
// two 16-byte chunks l/16 and 4 + l/16 of the 128-byte row. The K order this
// induces is the same for both operands, so the contraction is unchanged, and each
// 16-byte half is one whole 32-element block when the row holds fp4.
__device__ __forceinline__ v8i lds_frag(uint32_t addr_lo, uint32_t addr_hi, int imm) {
    v4i lo = *(lds_v4i_t*)(uintptr_t)(addr_lo + imm);
    v4i hi = *(lds_v4i_t*)(uintptr_t)(addr_hi + imm);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// D(16x16, fp32) += A(16x128, e4m3) * B(16x128, e4m3)^T. Lane l supplies row l%16,
// K-block l/16 of each operand and receives D[4*(l/16)+j][l%16] in element j.
// Same instruction as the reference's mfma1616128
// (include/ops/warp/register/tile/mma.cuh:112-125).
__device__ __forceinline__ v4f mfma_fp8_16x16x128(v8i a, v8i b, v4f c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// D(16x16, fp32) += X(16x128 e2m1, scale sx) * Y(16x128 e2m1, scale sy)^T: the FP4 form of the
// same instruction (cbsz = blgp = 4). Each lane holds 32 elements (16 bytes) of its row's K-block
// l/16 and supplies the e8m0 scale of exactly that block in bits [7:0] of sx / sy. The builtin
// takes 8-dword operands of which the FP4 form reads the first four; the duplicate shuffle costs
// no instructions.
__device__ __forceinline__ v4f mfma_fp4(v4i x, v4i y, v4f c, int sx, int sy) {
    v8i x8 = __builtin_shufflevector(x, x, 0, 1, 2, 3, 0, 1, 2, 3);
    v8i y8 = __builtin_shufflevector(y, y, 0, 1, 2, 3, 0, 1, 2, 3);
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x8, y8, c, 4, 4, 0, sx, 0, sy);
}

// Uniform 16-byte read through the scalar cache (s_load_dwordx4); `p` must be wave-uniform and
// point to data written before this kernel started.
__device__ __forceinline__ v4i scalar_load_x4(const void* p) {
    v4i r;
    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(p) : "memory");
    return r;
}
// 16 consecutive floats (four s_load_dwordx4, one wait); same conditions, p 16-byte aligned.
__device__ __forceinline__ void scalar_load_f16(const float* p, float (&out)[16]) {
    v4i a, b, c, d;
    asm volatile(
        "s_load_dwordx4 %0, %4, 0x0\n\ts_load_dwordx4 %1, %4, 0x10\n\t"
        "s_load_dwordx4 %2, %4, 0x20\n\ts_load_dwordx4 %3, %4, 0x30\n\ts_waitcnt lgkmcnt(0)"
        : "=&s"(a), "=&s"(b), "=&s"(c), "=&s"(d) : "s"(p) : "memory");
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[i] = __int_as_float(a[i]);
        out[4 + i] = __int_as_float(b[i]);
        out[8 + i] = __int_as_float(c[i]);
        out[12 + i] = __int_as_float(d[i]);
    }
}
__device__ __forceinline__ int scalar_load_x1(const void* p) {
    int r;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r) : "s"(p) : "memory");
    return r;
}

// Global stores the compiler does not see. On this ISA loads and stores share one counter but
// complete out of order with respect to each other, so a compiler that sees both kinds pending
// waits for all of them (vmcnt(0)) before the first use of any loaded register; kernels that
// keep register loads in flight across an epilogue issue the epilogue's stores through these.
// (A store of more than 8 bytes reads its data registers for two more cycles after issue: a VALU
// instruction that overwrites them must keep that distance. The compiler spaces its own stores; for
// this one, which it cannot see, the two wait states are part of the statement.)
__device__ __forceinline__ void store_global_b128(void* p, v4i v) {
    asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_global_b32(void* p, uint32_t v) {
    asm volatile("global_store_dword %0, %1, off" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_global_b8(void* p, uint32_t v) {
    asm volatile("global_store_byte %0, %1, off" ::"v"(p), "v"(v) : "memory");
}

// Same MFMA with the accumulator tied in place in an accumulation register (AGPR).
// Used by the hand-scheduled kernels, where the register allocator must not move
// accumulators between register files. The compiler does not see the instruction's
// hazards: accumulators may be read by other instructions only after
// mfma_drain() (the operands here come from LDS reads, which need no extra spacing).
__device__ __forceinline__ void mfma_fp8_16x16x128_acc(v4f& acc, const v8i& a, const v8i& b) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// Wait states between the last MFMA and the first read of its result by a
// non-MFMA instruction (the longest case on this ISA is 18 cycles for a 16-pass MFMA).
__device__ __forceinline__ void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 7" ::: "memory"); }
// mfma_drain() for accumulators written by the asm MFMA statements: every later read of `acc`
// depends on the drain. Reads of registers are not memory operations, and the compiler, which sees
// no hazard behind those statements, may otherwise move them above it, next to the MFMAs.
// (Volatile asm statements keep their order; each accumulator passes through one.)
template <int M, int N>
__device__ __forceinline__ void mfma_drain_agpr(v4f (&acc)[M][N]) {
    mfma_drain();
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int n = 0; n < N; ++n) asm volatile("" : "+a"(acc[m][n]));
}
template <int M, int N>
__device__ __forceinline__ void mfma_drain_vgpr(v4f (&acc)[M][N]) {
    mfma_drain();
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int n = 0; n < N; ++n) asm volatile("" : "+v"(acc[m][n]));
}

// Two fp32 -> packed bf16 (round to nearest even); `lo` goes to bits [15:0].
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    v2f f = {lo, hi};
    v2bf h = __builtin_convertvector(f, v2bf);
    return __builtin_bit_cast(uint32_t, h);
}

// Workgroup order. Hardware hands consecutive workgroup ids to the 8 XCDs round
// robin. `xcd_chunk_order` regroups ids so that each XCD (own L2) owns runs of
// `chunk` consecutive logical ids (cf. chiplet_transform_chunked,
// include/common/util.cuh:78-101); `grouped_raster` then walks the tile grid in
// column-major groups of `group_m` tile rows so that a run of `chunk` ids is a
// compact 2-D patch of C sharing A/B panels in that L2.
__device__ __forceinline__ int xcd_chunk_order(int wg, int num_wg, int chunk) {
    const int span = kNumXcd * chunk;
    const int full = (num_wg / span) * span;
    if (wg >= full) return wg;
    const int xcd = wg % kNumXcd;
    const int local = wg / kNumXcd;
    return (local / chunk) * span + xcd * chunk + (local % chunk);
}

__device__ __forceinline__ void grouped_raster(int id, int tiles_m, int tiles_n, int group_m,
                                               int& pm, int& pn) {
    const int per_group = group_m * tiles_n;
    const int group = id / per_group;
    const int first_m = group * group_m;
    const int gsize = min(tiles_m - first_m, group_m);
    const int in_group = id - group * per_group;
    pm = first_m + in_group % gsize;
    pn = in_group / gsize;
    // odd groups run right to left: the B panels the previous group used last are the first ones
    // the next group asks for, while they are still in the memory-side cache
    if (group & 1) pn = tiles_n - 1 - pn;
}

// grouped_raster inside bands of `band_n` tile columns (the last band takes the remainder): a run
// of 256 ids then covers a squarish 16 x 16 patch of tiles whose B panels stay in the memory-side
// cache while the band's tile rows stream past, instead of a stripe across all columns.
__device__ __forceinline__ void banded_raster(int id, int tiles_m, int tiles_n, int group_m, int band_n,
                                              int& pm, int& pn) {
    const int bands = max(1, tiles_n / band_n);
    const int per_band = tiles_m * band_n;
    const int band = min(id / per_band, bands - 1);
    const int first_n = band * band_n;
    const int width = band < bands - 1 ? band_n : tiles_n - first_n;
    grouped_raster(id - band * per_band, tiles_m, width, group_m, pm, pn);
    pn += first_n;
}

}  // namespace hk
