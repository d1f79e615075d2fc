// Per-point code arithmetic, usable from device code and from a host-side check build.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define PTV3_HD __host__ __device__ __forceinline__
#else
#define PTV3_HD static inline
#endif

namespace ptv3 {

// Spread the low 16 bits of v so that bit i lands on bit 3*i.
PTV3_HD uint64_t spread3(uint32_t v) {
    uint64_t x = v & 0xffffu;
    x = (x | (x << 32)) & 0x001f00000000ffffull;
    x = (x | (x << 16)) & 0x001f0000ff0000ffull;
    x = (x | (x << 8)) & 0x100f00f00f00f00full;
    x = (x | (x << 4)) & 0x10c30c30c30c30c3ull;
    x = (x | (x << 2)) & 0x1249249249249249ull;
    return x;
}

PTV3_HD uint64_t interleave(uint32_t a, uint32_t b, uint32_t c) {
    return (spread3(a) << 2) | (spread3(b) << 1) | spread3(c);
}

// Skilling's axes-to-transpose on three `depth`-bit words, then Gray decode of the
// interleaved word (prefix XOR from the top bit).
PTV3_HD uint64_t hilbert3(uint32_t x0, uint32_t x1, uint32_t x2, int depth) {
    for (int q = depth - 1; q > 0; --q) {   // level 0 has no lower bits to edit
        const uint32_t Q = 1u << q, P = Q - 1u;
        // axis 0: invert its own lower bits when its bit is set
        x0 ^= (x0 & Q) ? P : 0u;
        // axis 1
        {
            const uint32_t t = (x0 ^ x1) & P;
            const bool on = x1 & Q;
            x0 ^= on ? P : t;
            x1 ^= on ? 0u : t;
        }
        // axis 2
        {
            const uint32_t t = (x0 ^ x2) & P;
            const bool on = x2 & Q;
            x0 ^= on ? P : t;
            x2 ^= on ? 0u : t;
        }
    }
    uint64_t h = interleave(x0, x1, x2);
    h ^= h >> 1;
    h ^= h >> 2;
    h ^= h >> 4;
    h ^= h >> 8;
    h ^= h >> 16;
    h ^= h >> 32;
    return h;
}


// order id: bit 0 = swap x/y ("-trans"), ids 2..3 = Hilbert.
PTV3_HD uint64_t curve_code(int id, uint32_t x, uint32_t y, uint32_t z, int depth) {
    const uint32_t a = (id & 1) ? y : x;
    const uint32_t b = (id & 1) ? x : y;
    return (id < 2) ? interleave(a, b, z) : hilbert3(a, b, z, depth);
}

}  // namespace ptv3
