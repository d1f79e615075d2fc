// Half-precision building blocks shared by the patch attention kernels (forward and backward):
// the 32x32x16 MFMA per 16-bit type, packing, and the key-axis permutation of transposed tiles.
#pragma once
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int HD = 16;             // head dim
constexpr int ATT_THREADS = 512;   // 8 waves, two work-groups per CU -> 4 waves per SIMD
constexpr int ATT_WAVES = ATT_THREADS / PTV3_WAVE;
constexpr int VT_PAD_BYTES = 16;   // skews V^T rows across LDS banks

// Attention dropout (model.py:470, :480): probability (head, query slot q, key slot k) is kept when a 32-bit
// hash of (seed, head, q, k) reaches the threshold p * 2^32; forward and backward kernels recompute the same
// bits instead of storing a mask. hq = the part that does not depend on the key.
__device__ __forceinline__ uint32_t drop_hq(uint32_t seed, uint32_t head, uint32_t q) {
    return (q * 0x9E3779B1u) ^ ((head + 1u) * 0xC2B2AE3Du) ^ seed;
}
__device__ __forceinline__ bool drop_keep(uint32_t hq, uint32_t k, uint32_t threshold) {
    uint32_t x = hq ^ ((k + 0x7F4A7C15u) * 0x85EBCA77u);
    x ^= x >> 16;
    x *= 0x7FEB352Du;
    x ^= x >> 15;
    x *= 0x846CA68Bu;
    x ^= x >> 16;
    return x >= threshold;
}
static inline uint32_t drop_threshold(float p) {
    const double t = (double)p * 4294967296.0;
    return t >= 4294967295.0 ? 0xFFFFFFFFu : (uint32_t)t;
}
struct Dropout {
    uint32_t seed, threshold;   // threshold 0: no dropout
    float inv_keep;             // 1 / (1 - p)
};

template <typename T> struct Half;
template <> struct Half<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        f16x2 h = __builtin_convertvector(f, f16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ uint16_t one() { return 0x3C00; }
    // |score| (log2 units) up to which 2^score needs no shift: normal fp16 numbers are 2^-14 .. 2^15
    static __device__ __forceinline__ float plain_limit() { return 14.f; }
};
template <> struct Half<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        bf16x2 h = __builtin_convertvector(f, bf16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ uint16_t one() { return 0x3F80; }
    // bf16 has fp32's exponent range; 1024 keys of 2^100 still sum within fp32
    static __device__ __forceinline__ float plain_limit() { return 100.f; }
};

// position of key kk (0..31) inside its 32-key block of the transposed V tile: the keys a
// lane of half h holds in result registers 0..15 are 8*(v/4) + 4*h + v%4.
__device__ __forceinline__ int vt_pos(int kk) {
    return ((kk >> 2) & 1) * 16 + (kk >> 3) * 4 + (kk & 3);
}

template <typename T>
__device__ __forceinline__ float sum_sq8(u32x4 w) {
    typedef typename Half<T>::v8 v8;
    const v8 h = __builtin_bit_cast(v8, w);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = fmaf((float)h[i], (float)h[i], s);
    return s;
}

template <typename T>
__device__ __forceinline__ u32x4 scale8(u32x4 w, float c) {
    typedef typename Half<T>::v8 v8;
    const v8 h = __builtin_bit_cast(v8, w);
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = Half<T>::pack2((float)h[2 * i] * c, (float)h[2 * i + 1] * c);
    return r;
}

}  // namespace
