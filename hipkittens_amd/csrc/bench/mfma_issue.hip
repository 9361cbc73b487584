// Bench-only probe, built into libhk355_bench.so (not part of libhk355.so or of its C ABI; only bench.py
// loads it): how many other instructions one wave per SIMD can issue beside each MFMA before the MFMAs slow
// down. A register-only loop (all-zero operands: no power limit) of independent MFMAs, each followed by KOPS
// instructions of one kind; the kernel reports the shader clocks of its first wave. The hand-placed schedules
// of the tile kernels are sized by these figures (how many LDS reads, loads and scalar instructions an MFMA
// slot can carry). No counterpart in the reference.
#include "../hk_device.h"

namespace hk {

typedef float v16f __attribute__((ext_vector_type(16)));

// MODE 0: v_mfma_f32_16x16x128_f8f6f4 on FP8 operands (8 passes); 1: the scaled form on FP4 operands (4 passes);
// 2: v_mfma_scale_f32_32x32x64_f8f6f4 on FP4 operands (8 passes). KIND 0: v_add_u32 on registers of their
// own; 1: s_add_u32; 2: ds_read_b128 (64 lanes x 16 bytes).
template <int MODE, int KIND, int KOPS>
__global__ __launch_bounds__(256) void mfma_issue_kernel(const int* __restrict__ pattern, long long* __restrict__ out,
                                                         int iters) {
    __shared__ int lds[4096];
    lds[threadIdx.x] = 0;
    __syncthreads();
    v8i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            a[i][j] = pattern[(threadIdx.x * 8 + i * 64 + j) & 1023];
            b[i][j] = pattern[(threadIdx.x * 8 + i * 64 + j + 517) & 1023];
        }
    const int sc = pattern[threadIdx.x & 1023] & 0x7f7f7f7f;
    unsigned x[8] = {threadIdx.x, 1, 2, 3, 4, 5, 6, 7};
    unsigned sr[8] = {0, 1, 2, 3, 4, 5, 6, 7};
    const unsigned la = (unsigned)(uintptr_t)lds + (threadIdx.x & 63) * 16;
    v4i ld[KIND == 2 && KOPS > 0 ? KOPS : 1];
    auto others = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < KOPS; ++k) {
            if (KIND == 0) asm volatile("v_add_u32 %0, %0, 1" : "+v"(x[k]));
            else if (KIND == 1) asm volatile("s_add_u32 %0, %0, 1" : "+s"(sr[k]));
            else if constexpr (KIND == 2) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ld[k]) : "v"(la), "n"(k * 1024));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    long long t0, t1;
    float s = 0.f;
    if constexpr (MODE == 2) {
        v16f acc[12];   // (sixteen would take every register of the wave)
#pragma unroll
        for (int i = 0; i < 12; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
        t0 = clock64();
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 12; ++i) {
                acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 0, sc, 0, sc);
                others();
            }
        }
        t1 = clock64();
#pragma unroll
        for (int i = 0; i < 12; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) s += acc[i][j];
    } else {
        v4f acc[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
        t0 = clock64();
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                if (MODE == 0)
                    acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0, 0, 0, 0);
                else
                    acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 0, sc, 0, sc);
                others();
            }
        }
        t1 = clock64();
#pragma unroll
        for (int i = 0; i < 32; ++i) s += acc[i].x + acc[i].y + acc[i].z + acc[i].w;
    }
    // keep every result alive (the comparisons never hold)
    unsigned t = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) t += x[k] + sr[k];
    if constexpr (KIND == 2) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int k = 0; k < KOPS; ++k) t += (unsigned)ld[k].x;
    }
    if (s == 1.2345f || t == 0xdeadbeefu) out[1] = 1;
    if (threadIdx.x == 0 && blockIdx.x == 0) out[0] = t1 - t0;
}

template <int MODE, int KIND>
static int launch_issue(int kops, const int* pattern, long long* out, int iters, hipStream_t s) {
#define HK_ISSUE_CASE(K)                                                                                          \
    case K: hipLaunchKernelGGL((mfma_issue_kernel<MODE, KIND, K>), dim3(256), dim3(256), 0, s, pattern, out, iters); break;
    if constexpr (KIND == 2) {   // three 1 KiB reads per MFMA already exceed what the LDS delivers
        switch (kops) {
            HK_ISSUE_CASE(0) HK_ISSUE_CASE(1) HK_ISSUE_CASE(2) HK_ISSUE_CASE(3)
            default: return -2;
        }
    } else {
        switch (kops) {
            HK_ISSUE_CASE(0) HK_ISSUE_CASE(1) HK_ISSUE_CASE(2) HK_ISSUE_CASE(3) HK_ISSUE_CASE(4) HK_ISSUE_CASE(5) HK_ISSUE_CASE(6)
            default: return -2;
        }
    }
#undef HK_ISSUE_CASE
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace hk

// pattern: 1024 device ints (operand bits; zeros keep the clock up); out: 2 device int64, out[0] receives the
// shader clocks the first wave spent in its loop of iters x MFMAS MFMAs (MFMAS = 32, or 12 for mode 2).
// mode 0..2, kind 0..2, kops 0..6 (kind 2: at most 3): see the kernel.
extern "C" int hkbench_mfma_issue(const void* pattern, void* out, int mode, int kind, int kops, int iters, void* stream) {
    using namespace hk;
    if (!pattern || !out) return -1;
    if (mode < 0 || mode > 2 || kind < 0 || kind > 2 || kops < 0 || kops > 6 || (kind == 2 && kops > 3) || iters <= 0) return -2;
    hipStream_t s = (hipStream_t)stream;
    const int* p = (const int*)pattern;
    long long* o = (long long*)out;
#define HK_ISSUE_MODE(M)                                              \
    case M:                                                           \
        if (kind == 0) return launch_issue<M, 0>(kops, p, o, iters, s); \
        if (kind == 1) return launch_issue<M, 1>(kops, p, o, iters, s); \
        return launch_issue<M, 2>(kops, p, o, iters, s);
    switch (mode) {
        HK_ISSUE_MODE(0) HK_ISSUE_MODE(1) HK_ISSUE_MODE(2)
    }
#undef HK_ISSUE_MODE
    return -2;
}
