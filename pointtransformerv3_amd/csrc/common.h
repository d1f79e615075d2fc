// Shared helpers for the gfx950 kernels of libptv3_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>

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

// More than 64 KB of dynamic LDS has to be allowed per kernel, and the runtime keeps that attribute per device.
// A launcher keeps one LdsGrant per kernel instantiation (a function-local static): the largest size allowed so
// far on each device. ptv3_allow_lds raises it for the current device when `lds` exceeds it; 0 or a hipError_t.
constexpr int PTV3_MAX_DEVICES = 64;
struct LdsGrant {
    std::atomic<size_t> bytes[PTV3_MAX_DEVICES];
};
static inline int ptv3_allow_lds(const void* kern, size_t lds, LdsGrant& grant) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const bool tracked = dev >= 0 && dev < PTV3_MAX_DEVICES;
    if (tracked && lds <= grant.bytes[dev].load(std::memory_order_acquire)) return 0;
    static std::mutex mu;   // the slow path: set the attribute and record it as one step
    std::lock_guard<std::mutex> lock(mu);
    if (tracked && lds <= grant.bytes[dev].load(std::memory_order_relaxed)) return 0;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    if (tracked) grant.bytes[dev].store(lds, std::memory_order_release);
    return 0;
}

// Work-groups are dealt to the 8 XCDs round-robin in launch order, and every XCD has an L2 of its own.
// Launch index (or persistent-loop index, with a grid that is a multiple of 8) -> item such that each XCD
// works through one contiguous eighth of the items: neighbours in item order, which read the same cache lines
// (the heads of a sequence, the column blocks of one row tile), meet in one L2 at about the same time.
__device__ __forceinline__ int xcd_chunked_id(int bid, int total) {
    const int xcd = bid & 7, slot = bid >> 3;
    const int per = total >> 3, rem = total & 7;
    return xcd * per + min(xcd, rem) + slot;
}
