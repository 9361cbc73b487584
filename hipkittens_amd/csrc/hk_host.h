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

}  // namespace hk
