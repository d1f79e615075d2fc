// Shared helpers for the gfx950 kernels of libptv3_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ptv3_hip.h"

#define PTV3_WAVE 64

// Launch-error check: returns the hipError_t (> 0) to the C caller.
#define PTV3_RETURN_LAUNCH()                         \
    do {                                             \
        hipError_t e__ = hipGetLastError();          \
        return e__ == hipSuccess ? PTV3_OK : (int)e__; \
    } while (0)

static inline int64_t ptv3_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t ptv3_align256(size_t v) { return (v + 255) & ~(size_t)255; }
