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

// Up to 10 bits per axis the 30 code bits fit one 32-bit word: half the work of the 64-bit path on a 32-bit ALU.
PTV3_HD uint32_t spread3_10(uint32_t v) {
    uint32_t x = v & 0x3ffu;
    x = (x | (x << 16)) & 0x030000ffu;
    x = (x | (x << 8)) & 0x0300f00fu;
    x = (x | (x << 4)) & 0x030c30c3u;
    x = (x | (x << 2)) & 0x09249249u;
    return x;
}

PTV3_HD uint32_t interleave_10(uint32_t a, uint32_t b, uint32_t c) {
    return (spread3_10(a) << 2) | (spread3_10(b) << 1) | spread3_10(c);
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
    if (depth <= 10) {
        uint32_t g = interleave_10(x0, x1, x2);
        g ^= g >> 1;
        g ^= g >> 2;
        g ^= g >> 4;
        g ^= g >> 8;
        g ^= g >> 16;
        return g;
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


// Inverse of spread3: gather bits 0, 3, 6, ... of x into the low 16 bits.
PTV3_HD uint32_t compact3(uint64_t x) {
    x &= 0x1249249249249249ull;
    x = (x | (x >> 2)) & 0x10c30c30c30c30c3ull;
    x = (x | (x >> 4)) & 0x100f00f00f00f00full;
    x = (x | (x >> 8)) & 0x001f0000ff0000ffull;
    x = (x | (x >> 16)) & 0x001f00000000ffffull;
    x = (x | (x >> 32)) & 0xffffull;
    return (uint32_t)x;
}

// Inverse of hilbert3: Gray encode, de-interleave, then undo Skilling's edits from the lowest level up.
PTV3_HD void hilbert3_inverse(uint64_t h, int depth, uint32_t& x0, uint32_t& x1, uint32_t& x2) {
    const uint64_t g = h ^ (h >> 1);
    x0 = compact3(g >> 2);
    x1 = compact3(g >> 1);
    x2 = compact3(g);
    for (int q = 1; q < depth; ++q) {
        const uint32_t Q = 1u << q, P = Q - 1u;
        {
            const uint32_t t = (x0 ^ x2) & P;
            const bool on = x2 & Q;
            x0 ^= on ? P : t;
            x2 ^= on ? 0u : t;
        }
        {
            const uint32_t t = (x0 ^ x1) & P;
            const bool on = x1 & Q;
            x0 ^= on ? P : t;
            x1 ^= on ? 0u : t;
        }
        x0 ^= (x0 & Q) ? P : 0u;
    }
}

// order id: bit 0 = swap x/y ("-trans"), ids 2..3 = Hilbert.
PTV3_HD uint64_t curve_code(int id, uint32_t x, uint32_t y, uint32_t z, int depth) {
    const uint32_t a = (id & 1) ? y : x;
    const uint32_t b = (id & 1) ? x : y;
    if (id >= 2) return hilbert3(a, b, z, depth);
    return depth <= 10 ? (uint64_t)interleave_10(a, b, z) : interleave(a, b, z);
}

// Inverse of curve_code on a code below 2^(3 depth).
PTV3_HD void curve_point(int id, uint64_t c, int depth, uint32_t& x, uint32_t& y, uint32_t& z) {
    uint32_t a, b;
    if (id < 2) {
        a = compact3(c >> 2);
        b = compact3(c >> 1);
        z = compact3(c);
    } else {
        hilbert3_inverse(c, depth, a, b, z);
    }
    x = (id & 1) ? b : a;
    y = (id & 1) ? a : b;
}

}  // namespace ptv3
