// Submanifold sparse convolution forward as an output-stationary implicit GEMM over the
// neighbour map.
//
// Replaces spconv.SubMConv3d.forward at the reference call sites model.py:546-552 (xCPE,
// 3x3x3, bias) and :767-774 (stem, 5x5x5, no bias).
//
// Half-precision kernel: a workgroup owns VOX voxels x COUT_TILE output channels and keeps
// that block of the output in MFMA accumulators for the whole tap loop, so there is no
// atomic scatter and every output element is written once. Per (tap, 64-channel slice):
//   * the W[couts, tap, cin-slice] tile goes through LDS (shared by the 4 waves)
//   * neighbour rows are gathered straight from global memory into MFMA operand registers:
//     in v_mfma_f32_32x32x16 a lane's operand is 8 consecutive input channels of one voxel,
//     i.e. one 16-byte load from the gathered row
//   * a wave skips a tap when none of its voxels has that neighbour; the workgroup skips
//     staging the weights when no wave needs them
// The product is taken transposed (rows = output channels, columns = voxels) so a lane ends
// up holding 4 consecutive output channels of one voxel per register group and stores 8 B.
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

template <typename T> struct HalfOps;
template <> struct HalfOps<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ float to_float(_Float16 v) { return (float)v; }
};
template <> struct HalfOps<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ float to_float(__bf16 v) { return (float)v; }
};

constexpr int CONV_THREADS = 256;
constexpr int CONV_WAVES = CONV_THREADS / PTV3_WAVE;
constexpr int KC = 64;           // input-channel slice staged per step
constexpr int W_PAD = 8;         // halfs of padding per LDS weight row

// MT: 32-voxel tiles per wave; NT: 32-channel output tiles per workgroup.
template <typename T, int MT, int NT>
__global__ __launch_bounds__(CONV_THREADS) void subm_conv_half_kernel(
    const T* __restrict__ feat, int64_t n, int cin, const int32_t* __restrict__ nbr, int taps,
    const T* __restrict__ weight, const T* __restrict__ bias, int cout, T* __restrict__ out) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int VOX = CONV_WAVES * MT * 32;
    constexpr int COUT_TILE = NT * 32;
    __shared__ __align__(16) T w_lds[COUT_TILE][KC + W_PAD];

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int64_t vox0 = (int64_t)blockIdx.x * VOX + wave * (MT * 32);
    const int cout0 = blockIdx.y * COUT_TILE;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    int64_t vox[MT];
#pragma unroll
    for (int a = 0; a < MT; ++a) vox[a] = vox0 + a * 32 + col;

    for (int t = 0; t < taps; ++t) {
        int32_t src[MT];
        bool wave_any = false;
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            src[a] = vox[a] < n ? nbr[vox[a] * taps + t] : -1;
            wave_any |= (__ballot(src[a] >= 0) != 0);
        }
        if (!__syncthreads_or(wave_any)) continue;   // block-uniform: nobody has this tap

        for (int c0 = 0; c0 < cin; c0 += KC) {
            const int kc = min(KC, cin - c0);   // multiple of 16
            __syncthreads();   // previous slice fully consumed
            // stage W[cout0.., t, c0..c0+kc) as [cout][cin]; 16-byte pieces
            const int pieces = kc / 8;
            for (int e = tid; e < COUT_TILE * pieces; e += CONV_THREADS) {
                const int co = e / pieces, pc = e % pieces;
                u32x4 w = {0, 0, 0, 0};
                if (cout0 + co < cout)
                    w = *(const u32x4*)(weight + ((int64_t)(cout0 + co) * taps + t) * cin + c0 + pc * 8);
                *(u32x4*)&w_lds[co][pc * 8] = w;
            }
            __syncthreads();
            if (wave_any) {
                for (int k0 = 0; k0 < kc; k0 += 16) {
                    v8 xfrag[MT];
#pragma unroll
                    for (int a = 0; a < MT; ++a) {
                        u32x4 x = {0, 0, 0, 0};
                        if (src[a] >= 0) x = *(const u32x4*)(feat + (int64_t)src[a] * cin + c0 + k0 + hf * 8);
                        xfrag[a] = __builtin_bit_cast(v8, x);
                    }
#pragma unroll
                    for (int b = 0; b < NT; ++b) {
                        const v8 wfrag = __builtin_bit_cast(v8, *(const u32x4*)&w_lds[b * 32 + col][k0 + hf * 8]);
#pragma unroll
                        for (int a = 0; a < MT; ++a) acc[a][b] = HalfOps<T>::mfma(wfrag, xfrag[a], acc[a][b]);
                    }
                }
            }
        }
    }

    // acc[a][b][v]: output channel cout0 + b*32 + 8*(v/4) + 4*hf + v%4 of voxel vox[a]
#pragma unroll
    for (int a = 0; a < MT; ++a) {
        if (vox[a] >= n) continue;
#pragma unroll
        for (int b = 0; b < NT; ++b) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int co = cout0 + b * 32 + 8 * g + 4 * hf;
                if (co >= cout) continue;
                float r[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    r[q] = acc[a][b][4 * g + q] + (bias ? HalfOps<T>::to_float(bias[co + q]) : 0.f);
                u32x2 pk = {HalfOps<T>::pack2(r[0], r[1]), HalfOps<T>::pack2(r[2], r[3])};
                *(u32x2*)(out + vox[a] * cout + co) = pk;
            }
        }
    }
}

// fp32: one thread per (voxel, output channel); a wave shares the voxel when cout >= 64.
__global__ __launch_bounds__(256) void subm_conv_f32_kernel(
    const float* __restrict__ feat, int64_t n, int cin, const int32_t* __restrict__ nbr, int taps,
    const float* __restrict__ weight, const float* __restrict__ bias, int cout,
    float* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * cout) return;
    const int64_t i = e / cout;
    const int co = (int)(e - i * cout);
    float acc = bias ? bias[co] : 0.f;
    for (int t = 0; t < taps; ++t) {
        const int32_t src = nbr[i * taps + t];
        if (src < 0) continue;
        const float* x = feat + (int64_t)src * cin;
        const float* w = weight + ((int64_t)co * taps + t) * cin;
        float part = 0.f;
        for (int c = 0; c < cin; ++c) part = fmaf(x[c], w[c], part);
        acc += part;
    }
    out[e] = acc;
}

template <typename T, int MT, int NT>
void launch_half(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps,
                 const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    constexpr int VOX = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    dim3 grid((unsigned)ptv3_ceil_div(n, VOX), (unsigned)ptv3_ceil_div(cout, COUT_TILE));
    hipLaunchKernelGGL((subm_conv_half_kernel<T, MT, NT>), grid, dim3(CONV_THREADS), 0, stream,
                       (const T*)feat, n, cin, nbr, taps, (const T*)weight, (const T*)bias, cout,
                       (T*)out);
}

template <typename T>
void dispatch_half(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps,
                   const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    // Wide voxel tiles while there are enough voxels to fill 256 CUs; narrow ones otherwise.
    const bool big = n >= 64 * 1024;
    if (cout <= 32) {
        if (big) launch_half<T, 2, 1>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
        else launch_half<T, 1, 1>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
    } else {
        if (big) launch_half<T, 2, 2>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
        else launch_half<T, 1, 2>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
    }
}

}  // namespace

extern "C" int ptv3_subm_conv_fwd(const void* feat, int dtype, int64_t n, int cin,
                                  const int32_t* nbr, int taps, const void* weight,
                                  const void* bias, int cout, void* out, void* stream_) {
    if (n < 0 || cin < 1 || cout < 1 || taps < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!feat || !nbr || !weight || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F32) {
        hipLaunchKernelGGL(subm_conv_f32_kernel, dim3((unsigned)ptv3_ceil_div(n * cout, 256)), dim3(256),
                           0, stream, (const float*)feat, n, cin, nbr, taps, (const float*)weight,
                           (const float*)bias, cout, (float*)out);
        PTV3_RETURN_LAUNCH();
    }
    // operand registers are 8-channel pieces of 16-channel steps; stores are 4-channel pieces
    if (cin % 16 != 0 || cout % 4 != 0) return PTV3_ESHAPE;
    if (dtype == PTV3_F16)
        dispatch_half<_Float16>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
    else
        dispatch_half<__bf16>(feat, n, cin, nbr, taps, weight, bias, cout, out, stream);
    PTV3_RETURN_LAUNCH();
}
