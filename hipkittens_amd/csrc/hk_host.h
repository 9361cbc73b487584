// Host-side helpers shared by the launchers.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

namespace hk {

// One bit per device ordinal: has this launcher's kernel been configured on that device?
struct DeviceOnce {
    std::atomic<uint64_t> done{0};
};

// Raises the dynamic-LDS limit of `kern` to `bytes` on the current device, once per device. The
// attribute belongs to the function as loaded on one device, so a process that drives several GPUs
// sets it on each. Safe to call from several threads: two callers that race both make the (idempotent)
// HIP call. Devices with an ordinal of 64 and more are configured on every call.
inline bool set_lds_limit_once(const void* kern, int bytes, DeviceOnce& once) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    const uint64_t bit = dev < 64 ? 1ull << dev : 0ull;
    if (once.done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    once.done.fetch_or(bit, std::memory_order_release);
    return true;
}

// Whether a GEMM's dimensions are beyond what the launchers' 32-bit arithmetic covers: a dimension of 2^30
// or more, or 2^31 and more tiles of 64 x 64 (tile counts and grid sizes are ints). Every public GEMM entry
// point refuses such a shape before it computes anything from it.
inline bool gemm_dims_too_large(int M, int N, int K) {
    if (M >= (1 << 30) || N >= (1 << 30) || K >= (1 << 30)) return true;
    if (M <= 0 || N <= 0) return false;
    return (((long long)M + 63) / 64) * (((long long)N + 63) / 64) >= (1ll << 31);
}

}  // namespace hk
