// cv_launch.h -- host-side launch helpers shared by the kernel launchers.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

namespace cv {

constexpr int kMaxDevices = 64;

// index of the current device, or -1 when it cannot be cached (query failed / beyond the tables)
inline int currentDeviceSlot()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
    return dev;
}

// Workgroups of `Kernel` (threads per group, no dynamic LDS) resident at once on one compute unit
// of the current device.  The residency of a kernel on a device never changes, so it is queried
// once per (kernel, device); the cache is a table of atomics, and a lost race only repeats the
// (idempotent) query.
template <auto Kernel>
int residentBlocksPerCU(int threads)
{
    static std::atomic<int> cache[kMaxDevices];
    const int dev = currentDeviceSlot();
    if (dev >= 0) {
        const int v = cache[dev].load(std::memory_order_relaxed);
        if (v > 0) return v;
    }
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, Kernel, threads, 0) != hipSuccess || n < 1) n = 1;
    if (dev >= 0) cache[dev].store(n, std::memory_order_relaxed);
    return n;
}

// Raises the dynamic-LDS limit of `Kernel` on the current device, once per (kernel, device).
template <auto Kernel>
hipError_t allowDynamicLds(int bytes)
{
    static std::atomic<int> done[kMaxDevices];
    const int dev = currentDeviceSlot();
    if (dev >= 0 && done[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && dev >= 0) done[dev].store(bytes, std::memory_order_release);
    return e;
}

} // namespace cv
