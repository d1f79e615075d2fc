// Shared pieces of the row-tile kernels (fused MLP, fused block head / tail): a wave owns 32 rows,
// products are taken transposed with v_mfma_f32_32x32x16 so that every lane owns one row.
#pragma once
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct H16;
template <> struct H16<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ float round(float v) { return (float)(_Float16)v; }
    static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
    static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
};
template <> struct H16<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ float round(float v) { return (float)(__bf16)v; }
    static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(bf16x2, w)[0]; }
    static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(bf16x2, w)[1]; }
};

// position of hidden unit kk (0..31) of a 32-block in W2's LDS row: registers 0..15 of a lane of
// half h hold rows 8*(v/4) + 4*h + v%4 of the first product
__device__ __forceinline__ int perm32(int kk) { return ((kk >> 2) & 1) * 16 + (kk >> 3) * 4 + (kk & 3); }

// The exact (erf) GELU of nn.GELU for results that are stored in half precision:
//   x Phi(x) = max(x, 0) - |x| * erfc(|x| / sqrt 2) / 2,
// with log2(erfc(a / sqrt 2) / 2) as a polynomial of degree 7 in a = |x| (minimax on [0, 5.7]: |error| < 5.6e-6,
// that is 4e-6 relative in erfc, in the tail as well; beyond 5.7 the polynomial keeps falling, the term vanishes
// and no clamp is needed). Seven FMAs, one v_exp_f32, a max and an FMA: the Abramowitz-Stegun 7.1.26 form it
// replaces took 13 instructions and two transcendentals, and its 1 - (...) cancels in the negative tail.
// A non-finite input (a first-layer sum beyond the half-precision range, or NaN) gives NaN: the polynomial meets
// inf * 0. Clamping |x| would cost an instruction per element and, with min/max returning their non-NaN operand,
// swallow a NaN; torch's own CPU kernel returns NaN or the limit for +-inf depending on the machine's vector path.
// Over every finite fp16 input (a test passes them all through a kernel): rounded to fp16 the result differs from the correctly rounded
// GELU for 47 of 63487 inputs, by one ulp (461 with the 7.1.26 form); rounded to bf16 for 10 inputs with |x| < 8.
__device__ __forceinline__ float gelu_erf(float x) {
    const float a = fabsf(x);
    float p = fmaf(-1.771743957e-06f, a, 6.035297709e-05f);
    p = fmaf(p, a, -9.207596672e-04f);
    p = fmaf(p, a, 8.469257484e-03f);
    p = fmaf(p, a, -5.387924940e-02f);
    p = fmaf(p, a, -4.585495940e-01f);
    p = fmaf(p, a, -1.151212616e+00f);
    p = fmaf(p, a, -1.0f);
    return fmaf(-a, __builtin_amdgcn_exp2f(p), fmaxf(x, 0.f));
}

// GELU of two first-layer sums as the separate layers would have stored them: rounded to the storage type, passed
// through gelu_erf, rounded again and packed. For fp16 the rounded pair stays packed: the polynomial's FMAs read
// its halves directly (v_fma_mix_f32 converts on the way in), max(x, 0) is one packed instruction for the pair, and
// the only conversions left are the two packed ones (10.5 instructions per element instead of 12.5). Same operations
// on the same values as gelu_erf(round(x)): the same bits.
template <typename T> __device__ __forceinline__ uint32_t gelu_round_pack2(float x0, float x1) {
    return H16<T>::pack2(gelu_erf(H16<T>::round(x0)), gelu_erf(H16<T>::round(x1)));
}
template <> __device__ __forceinline__ uint32_t gelu_round_pack2<_Float16>(float x0, float x1) {
    const f32x2 f = {x0, x1};
    const f16x2 h = __builtin_convertvector(f, f16x2);
    const f16x2 zero = {(_Float16)0, (_Float16)0};
    const f16x2 m = __builtin_elementwise_max(h, zero);
    f32x2 r;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float a = (float)__builtin_fabsf16(h[k]);
        float p = fmaf(-1.771743957e-06f, a, 6.035297709e-05f);
        p = fmaf(p, a, -9.207596672e-04f);
        p = fmaf(p, a, 8.469257484e-03f);
        p = fmaf(p, a, -5.387924940e-02f);
        p = fmaf(p, a, -4.585495940e-01f);
        p = fmaf(p, a, -1.151212616e+00f);
        p = fmaf(p, a, -1.0f);
        r[k] = fmaf(-a, __builtin_amdgcn_exp2f(p), (float)m[k]);
    }
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(r, f16x2));
}

// d/dx of gelu_erf: Phi(x) + x phi(x); the erf approximation's exponential is phi's as well
__device__ __forceinline__ float gelu_erf_grad(float x) {
    const float z = fabsf(x) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
    float p = fmaf(1.061405429f, t, -1.453152027f);
    p = fmaf(p, t, 1.421413741f);
    p = fmaf(p, t, -0.284496736f);
    p = fmaf(p, t, 0.254829592f);
    const float e = __builtin_amdgcn_exp2f(-z * z * 1.4426950408889634f);
    const float erf_abs = fmaf(-p * t, e, 1.0f);
    return fmaf(x * 0.3989422804014327f, e, fmaf(copysignf(erf_abs, x), 0.5f, 0.5f));
}

}  // namespace
