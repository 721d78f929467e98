// Host-side helpers shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/coat_hip.h"

// Status of the launch just issued: COAT_OK or the (positive) hipError_t.
static inline int coat_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? COAT_OK : (int)e;
}
// Kernels move 16 bytes per lane; NULL (an optional output that is absent) counts as aligned.
static inline bool coat_aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
