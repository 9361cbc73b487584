// Bench-only calibration probe, built into libhk355_bench.so (not part of libhk355.so or of its
// C ABI; only bench.py loads it): sustained MFMA rate of this GPU from a register-only loop (no
// memory traffic), for a chosen operand bit pattern. On MI355X the matrix pipes are power limited, so the
// rate a GEMM can reach depends on how many operand bits toggle; this probe measures that ceiling
// for the data a benchmark actually uses. No counterpart in the reference.
#include "../hk_device.h"

namespace hk {

template <int FP4>
__global__ __launch_bounds__(512) void mfma_rate_kernel(const int* __restrict__ pattern, float* __restrict__ sink,
                                                        int iters) {
    // 8 waves per CU (two per SIMD), 32 independent accumulators per wave
    v8i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            a[i][j] = pattern[(threadIdx.x * 64 + i * 8 + j) & 16383];
            b[i][j] = pattern[(threadIdx.x * 64 + 32 + i * 8 + j + 7) & 16383];
        }
    v4f acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            if (FP4)
                acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 4, 4, 0,
                                                                           127, 0, 127);
            else
                acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0,
                                                                           0, 0, 0);
        }
    }
    v4f s = acc[0];
#pragma unroll
    for (int i = 1; i < 32; ++i) s += acc[i];
    sink[blockIdx.x * 512 + threadIdx.x] = s.x + s.y + s.z + s.w;
}

}  // namespace hk

// pattern: 16384 device ints used as operand bits (e.g. e4m3 bytes of the benchmark's data
// distribution); sink: >= blocks*512 device floats. Launches `blocks` workgroups of 8 waves running
// `iters` x 32 MFMAs (16x16x128, fp8 if fp4 == 0 else fp4) per wave. The caller times it;
// flops = blocks * 8 * iters * 32 * 65536.
extern "C" int hkbench_mfma_rate(const void* pattern, void* sink, int blocks, int iters, int fp4, void* stream) {
    using namespace hk;
    if (!pattern || !sink) return -1;
    if (blocks <= 0 || iters <= 0) return -2;
    if (fp4)
        hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(blocks), dim3(512), 0, (hipStream_t)stream, (const int*)pattern,
                           (float*)sink, iters);
    else
        hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(blocks), dim3(512), 0, (hipStream_t)stream, (const int*)pattern,
                           (float*)sink, iters);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}
