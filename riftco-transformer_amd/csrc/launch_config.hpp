// Launch-time configuration shared by the kernels that need more dynamic LDS
// than the default 64 KB.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

namespace rthip {

// Lets `kernel` use `bytes` of dynamic LDS on the current device.  The
// attribute belongs to the kernel's code object on ONE device, so a process
// that runs on several devices has to set it on each: `served` is the
// caller's set of devices (one bit each) on which this kernel already has it,
// a function-local static beside the launch.  Devices past 63 are configured
// on every launch.
inline hipError_t allow_dynamic_lds(const void* kernel, std::size_t bytes,
                                    std::atomic<std::uint64_t>& served) {
    int device = 0;
    if (const hipError_t error = hipGetDevice(&device); error != hipSuccess) {
        return error;
    }
    const std::uint64_t bit =
        device >= 0 && device < 64 ? std::uint64_t{1} << device : 0;
    if ((served.load(std::memory_order_acquire) & bit) != 0) {
        return hipSuccess;
    }
    const hipError_t error = hipFuncSetAttribute(
        kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(bytes));
    if (error == hipSuccess) {
        served.fetch_or(bit, std::memory_order_release);
    }
    return error;
}

}  // namespace rthip
