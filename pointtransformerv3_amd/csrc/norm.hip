// Row-wise LayerNorm fused with the residual additions that surround it in a PTv3 block.
//
// Replaces the nn.LayerNorm calls of model.py:554,557,572 together with the residual adds
// of :589,:594,:602. HBM-bound: every row is read once and written once (or twice when
// both the sum and its normalisation are needed). A row of C channels is spread over
// C/8 lanes (8 channels = one 16-byte load per lane in half precision), so a 64-lane wave
// normalises 64/(C/8) rows at a time and reductions are a few cross-lane steps.
//
//   mode 0: out0 = LN(x)
//   mode 1: out0 = res + LN(x)                      (cpe: shortcut + LN(Linear(conv)))
//   mode 2: out0 = x + res; out1 = LN(out0)         (shortcut + branch, then pre-norm)
//           with an optional per-channel `shift` added to the stored out0 only (the bias of the
//           GEMM that will accumulate onto out0), out1 is still LN(x + res)
//   mode 3: out0 = res + LN(x); out1 = LN2(out0)    (cpe residual, then the attention pre-norm)
// Intermediate results are rounded to the storage type exactly where separate kernels would
// have stored them, so fusing changes no value.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

template <typename T> struct Vec8 { T v[8]; };

template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&f)[8]) {
    const Vec8<T> r = *(const Vec8<T>*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)r.v[i];
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&f)[8]) {
    Vec8<T> r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = (T)f[i];
    *(Vec8<T>*)p = r;
}

template <typename T> __device__ __forceinline__ float round_to(float v) { return (float)(T)v; }

// statistics of 8 values per lane over the LPR lanes of a row
template <int LPR>
__device__ __forceinline__ void row_stats(const float (&v)[8], float eps, float& mean, float& rstd) {
    constexpr int C = 8 * LPR;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += v[i];
#pragma unroll
    for (int o = 1; o < LPR; o <<= 1) s += __shfl_xor(s, o, PTV3_WAVE);
    mean = s * (1.f / C);
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) q += (v[i] - mean) * (v[i] - mean);
#pragma unroll
    for (int o = 1; o < LPR; o <<= 1) q += __shfl_xor(q, o, PTV3_WAVE);
    rstd = rsqrtf(q * (1.f / C) + eps);
}

// LPR lanes per row, C = 8 * LPR channels.
template <typename T, int LPR, int MODE>
__global__ __launch_bounds__(256) void layer_norm_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const T* __restrict__ gamma,
    const T* __restrict__ beta, const T* __restrict__ gamma2, const T* __restrict__ beta2,
    const T* __restrict__ shift, int64_t n, float eps, T* __restrict__ out0, T* __restrict__ out1) {
    constexpr int C = 8 * LPR;
    constexpr int ROWS_PER_BLOCK = 256 / LPR;
    const int sub = threadIdx.x % LPR;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_BLOCK + threadIdx.x / LPR;
    const bool live = row < n;   // dead lanes still take part in the cross-lane sums
    const int64_t off = row * C + sub * 8;
    float v[8], r[8], g[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { v[i] = 0.f; r[i] = 0.f; }
    load8(gamma + sub * 8, g);
    load8(beta + sub * 8, b);
    if (live) {
        load8(x + off, v);
        if (MODE != 0) load8(res + off, r);
    }
    if (MODE == 2) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = round_to<T>(v[i] + r[i]);
        if (live) {
            if (shift) {
                float sh[8], w[8];
                load8(shift + sub * 8, sh);
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = v[i] + sh[i];
                store8(out0 + off, w);
            } else {
                store8(out0 + off, v);
            }
        }
    }
    float mean, rstd;
    row_stats<LPR>(v, eps, mean, rstd);
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (v[i] - mean) * rstd * g[i] + b[i];
    if (MODE == 1 || MODE == 3) {
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = round_to<T>(round_to<T>(y[i]) + r[i]);
    }
    if (MODE == 3) {
        if (live) store8(out0 + off, y);
        load8(gamma2 + sub * 8, g);
        load8(beta2 + sub * 8, b);
        row_stats<LPR>(y, eps, mean, rstd);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = (y[i] - mean) * rstd * g[i] + b[i];
    }
    if (live) store8((MODE >= 2) ? out1 + off : out0 + off, y);
}

// Any C: one wave per row, strided scalar accesses.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void layer_norm_generic_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const T* __restrict__ gamma,
    const T* __restrict__ beta, const T* __restrict__ shift, int64_t n, int c, float eps,
    T* __restrict__ out0, T* __restrict__ out1) {
    const int lane = threadIdx.x % PTV3_WAVE;
    const int64_t row = (int64_t)blockIdx.x * (256 / PTV3_WAVE) + threadIdx.x / PTV3_WAVE;
    if (row >= n) return;   // whole wave leaves together
    const T* xr = x + row * c;
    const T* rr = res ? res + row * c : nullptr;
    float s = 0.f;
    for (int i = lane; i < c; i += PTV3_WAVE) {
        float v = (float)xr[i];
        if (MODE == 2) {
            const T t = (T)(v + (float)rr[i]);
            out1[row * c + i] = t;   // parked in out1 until the statistics are known
            v = (float)t;
        }
        s += v;
    }
#pragma unroll
    for (int o = 1; o < PTV3_WAVE; o <<= 1) s += __shfl_xor(s, o, PTV3_WAVE);
    const float mean = s / c;
    float q = 0.f;
    for (int i = lane; i < c; i += PTV3_WAVE) {
        const float v = (MODE == 2 ? (float)out1[row * c + i] : (float)xr[i]) - mean;
        q += v * v;
    }
#pragma unroll
    for (int o = 1; o < PTV3_WAVE; o <<= 1) q += __shfl_xor(q, o, PTV3_WAVE);
    const float rstd = rsqrtf(q / c + eps);
    for (int i = lane; i < c; i += PTV3_WAVE) {
        const float v = MODE == 2 ? (float)out1[row * c + i] : (float)xr[i];
        float y = (v - mean) * rstd * (float)gamma[i] + (float)beta[i];
        if (MODE == 1) y = (float)(T)y + (float)rr[i];
        if (MODE == 2) out0[row * c + i] = (T)(v + (shift ? (float)shift[i] : 0.f));
        (MODE == 2 ? out1 : out0)[row * c + i] = (T)y;
    }
}

// Inference-mode BatchNorm1d followed (optionally) by exact GELU: y = act((x - mean) * rstd * gamma
// + beta), per channel, 8 channels per thread. The normalised value is rounded to the storage type
// before the activation, as two separate layers would round it.
__device__ __forceinline__ float gelu_exact(float x) {
    // 0.5 x (1 + erf(x / sqrt 2)); erf by Abramowitz-Stegun 7.1.26, |error| < 1.5e-7
    const float z = fabsf(x) * 0.70710678118654752f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
    float p = fmaf(1.061405429f, t, -1.453152027f);
    p = fmaf(p, t, 1.421413741f);
    p = fmaf(p, t, -0.284496736f);
    p = fmaf(p, t, 0.254829592f);
    const float e = __builtin_amdgcn_exp2f(-z * z * 1.4426950408889634f);
    const float erf_abs = fmaf(-p * t, e, 1.0f);
    const float half_x = 0.5f * x;
    return fmaf(copysignf(erf_abs, x), half_x, half_x);
}

template <typename T, typename S>
__global__ __launch_bounds__(256) void bn_act_kernel(const T* __restrict__ x, const S* __restrict__ mean,
                                                     const S* __restrict__ var, const T* __restrict__ gamma,
                                                     const T* __restrict__ beta, float eps, int act, int64_t n,
                                                     int c, T* __restrict__ out) {
    const int groups = c / 8;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * groups) return;
    const int ch = (int)(e % groups) * 8;
    float v[8], g[8], b[8], mu[8], va[8];
    load8(x + e * 8, v);
    load8(mean + ch, mu);
    load8(var + ch, va);
#pragma unroll
    for (int i = 0; i < 8; ++i) { g[i] = 1.f; b[i] = 0.f; }
    if (gamma) load8(gamma + ch, g);
    if (beta) load8(beta + ch, b);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float rstd = rsqrtf(va[i] + eps);
        float y = round_to<T>((v[i] - mu[i]) * rstd * g[i] + b[i]);
        v[i] = act == 1 ? gelu_exact(y) : y;
    }
    store8(out + e * 8, v);
}

template <typename T, int MODE>
void launch(const void* x, const void* res, const void* gamma, const void* beta, const void* gamma2,
            const void* beta2, const void* shift, int64_t n, int c, float eps, void* out0, void* out1,
            hipStream_t stream) {
#define PTV3_LN(LPR)                                                                            \
    hipLaunchKernelGGL((layer_norm_kernel<T, LPR, MODE>), dim3((unsigned)ptv3_ceil_div(n, 256 / LPR)), \
                       dim3(256), 0, stream, (const T*)x, (const T*)res, (const T*)gamma,       \
                       (const T*)beta, (const T*)gamma2, (const T*)beta2, (const T*)shift, n, eps, (T*)out0,  \
                       (T*)out1)
    switch (c) {
        case 32: PTV3_LN(4); break;
        case 64: PTV3_LN(8); break;
        case 128: PTV3_LN(16); break;
        case 256: PTV3_LN(32); break;
        case 512: PTV3_LN(64); break;
        default:
            if (MODE == 3) {   // two generic passes: out0 = res + LN(x), then out1 = LN2(out0)
                hipLaunchKernelGGL((layer_norm_generic_kernel<T, 1>), dim3((unsigned)ptv3_ceil_div(n, 4)),
                                   dim3(256), 0, stream, (const T*)x, (const T*)res, (const T*)gamma,
                                   (const T*)beta, (const T*)nullptr, n, c, eps, (T*)out0, (T*)nullptr);
                hipLaunchKernelGGL((layer_norm_generic_kernel<T, 0>), dim3((unsigned)ptv3_ceil_div(n, 4)),
                                   dim3(256), 0, stream, (const T*)out0, (const T*)nullptr, (const T*)gamma2,
                                   (const T*)beta2, (const T*)nullptr, n, c, eps, (T*)out1, (T*)nullptr);
            } else {
                constexpr int GM = MODE == 3 ? 0 : MODE;
                hipLaunchKernelGGL((layer_norm_generic_kernel<T, GM>), dim3((unsigned)ptv3_ceil_div(n, 4)),
                                   dim3(256), 0, stream, (const T*)x, (const T*)res, (const T*)gamma,
                                   (const T*)beta, (const T*)shift, n, c, eps, (T*)out0, (T*)out1);
            }
    }
#undef PTV3_LN
}

template <typename T>
void launch_mode(int mode, const void* x, const void* res, const void* gamma, const void* beta,
                 const void* gamma2, const void* beta2, const void* shift, int64_t n, int c, float eps,
                 void* out0, void* out1, hipStream_t stream) {
    if (mode == 0) launch<T, 0>(x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    else if (mode == 1) launch<T, 1>(x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    else if (mode == 2) launch<T, 2>(x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    else launch<T, 3>(x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
}

}  // namespace

extern "C" int ptv3_layer_norm(const void* x, const void* res, const void* gamma, const void* beta,
                               const void* gamma2, const void* beta2, const void* shift, int dtype,
                               int64_t n, int c, float eps, int mode, void* out0, void* out1,
                               void* stream_) {
    if (n < 0 || c < 1 || mode < 0 || mode > 3) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!x || !gamma || !beta || !out0) return PTV3_EINVAL;
    if (mode != 0 && !res) return PTV3_EINVAL;
    if (mode >= 2 && !out1) return PTV3_EINVAL;
    if (mode == 3 && (!gamma2 || !beta2)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F32)
        launch_mode<float>(mode, x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    else if (dtype == PTV3_F16)
        launch_mode<_Float16>(mode, x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    else
        launch_mode<__bf16>(mode, x, res, gamma, beta, gamma2, beta2, shift, n, c, eps, out0, out1, stream);
    PTV3_RETURN_LAUNCH();
}

template <typename T, typename S>
void launch_bn_act(const void* x, const void* mean, const void* var, const void* gamma, const void* beta, float eps,
                   int act, int64_t n, int c, void* out, hipStream_t stream) {
    hipLaunchKernelGGL((bn_act_kernel<T, S>), dim3((unsigned)ptv3_ceil_div(n * (c / 8), 256)), dim3(256), 0, stream,
                       (const T*)x, (const S*)mean, (const S*)var, (const T*)gamma, (const T*)beta, eps, act, n, c,
                       (T*)out);
}

extern "C" int ptv3_bn_act(const void* x, const void* running_mean, const void* running_var, int stats_f32,
                           const void* gamma, const void* beta, int dtype, int64_t n, int c, float eps, int act,
                           void* out, void* stream_) {
    if (n < 0 || c < 1 || act < 0 || act > 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (c % 8 != 0) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !running_mean || !running_var || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
#define PTV3_BN(T)                                                                                          \
    do {                                                                                                    \
        if (stats_f32) launch_bn_act<T, float>(x, running_mean, running_var, gamma, beta, eps, act, n, c, out, stream); \
        else launch_bn_act<T, T>(x, running_mean, running_var, gamma, beta, eps, act, n, c, out, stream);   \
    } while (0)
    if (dtype == PTV3_F32) PTV3_BN(float);
    else if (dtype == PTV3_F16) PTV3_BN(_Float16);
    else PTV3_BN(__bf16);
#undef PTV3_BN
    PTV3_RETURN_LAUNCH();
}
