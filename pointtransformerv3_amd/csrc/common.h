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

// Work-groups are dealt to the 8 XCDs round-robin in launch order, and every XCD has an L2 of its own.
// Launch index (or persistent-loop index, with a grid that is a multiple of 8) -> item such that each XCD
// works through one contiguous eighth of the items: neighbours in item order, which read the same cache lines
// (the heads of a sequence, the column blocks of one row tile), meet in one L2 at about the same time.
__device__ __forceinline__ int xcd_chunked_id(int bid, int total) {
    const int xcd = bid & 7, slot = bid >> 3;
    const int per = total >> 3, rem = total & 7;
    return xcd * per + min(xcd, rem) + slot;
}
