// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/coat_hip.h"

// Status of the launch just issued: COAT_OK or the (positive) hipError_t.
static inline int coat_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? COAT_OK : (int)e;
}
// Kernels move 16 bytes per lane; NULL (an optional output that is absent) counts as aligned.
static inline bool coat_aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// The current device's index, bounded for the per-device caches below (a process normally drives one GPU).
constexpr int kCoatMaxDevices = 64;
static inline int coat_device_index() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kCoatMaxDevices) return -1;
    return dev;
}
// Raises a kernel's dynamic-LDS limit once per device (the attribute is per device, the kernels are templates: each
// instantiation passes its own flag array).  The flags are atomics: host threads may enter an entry point together, and the
// worst that two of them can do is set the same attribute twice.
typedef std::atomic<bool> coat_device_flags[kCoatMaxDevices];
template <typename K> static inline int coat_allow_lds(K kernel, int bytes, std::atomic<bool>* done_per_device) {
    const int dev = coat_device_index();
    if (dev < 0) return COAT_EINVAL;
    if (!done_per_device[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return (int)e;
        done_per_device[dev].store(true, std::memory_order_release);
    }
    return COAT_OK;
}
