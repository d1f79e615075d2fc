// Half-precision (or transposed) copies of the fp32 master weights, all of them in one launch.
//
// Under autocast every nn.Linear and spconv.SubMConv3d of the model (model.py:366-367, :505-507, :546-553,
// :767-774) multiplies by a half-precision copy of its fp32 weight, and the input gradients multiply by the
// transpose: dx = dy W for a Linear, and for the submanifold convolution the same convolution with the
// taps mirrored and the two channel axes swapped. The optimizer rewrites all masters at once, so the copies
// are refreshed at once too: a table of jobs in device memory, a range of work-groups per job, one kernel.
// A work-group either converts 4096 consecutive elements, or moves one 64 x 64 tile of one tap through LDS
// so that both the fp32 reads and the transposed writes are contiguous.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

constexpr int CAST_CHUNK = 4096;   // elements of a plain job per work-group
constexpr int CAST_TILE = 64;      // tile edge of a mirrored job

template <typename T>
__device__ __forceinline__ T cast_to(float v) {
    return (T)v;
}
template <>
__device__ __forceinline__ __half cast_to<__half>(float v) {
    return __float2half(v);
}
template <>
__device__ __forceinline__ __hip_bfloat16 cast_to<__hip_bfloat16>(float v) {
    return __float2bfloat16(v);
}

template <typename T>
__global__ __launch_bounds__(256) void cast_params_kernel(const ptv3_cast_job* __restrict__ jobs, int n_jobs) {
    __shared__ float tile[CAST_TILE][CAST_TILE + 1];
    const int64_t blk = blockIdx.x;
    int lo = 0, hi = n_jobs - 1;   // the last job that starts at or before this work-group
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (jobs[mid].first_block <= blk) lo = mid;
        else hi = mid - 1;
    }
    const ptv3_cast_job job = jobs[lo];
    const int64_t local = blk - job.first_block;
    const float* __restrict__ src = job.src;
    T* __restrict__ dst = (T*)job.dst;
    const int tid = threadIdx.x;
    const int a = job.a, b = job.b, c = job.c;
    if (!job.mirror) {
        const int64_t total = (int64_t)a * b * c;
        const int64_t base = local * CAST_CHUNK;
        const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
#pragma unroll
        for (int k = 0; k < CAST_CHUNK / 1024; ++k) {
            const int64_t i = base + (int64_t)(k * 256 + tid) * 4;
            if (aligned && i + 3 < total) {
                const float4 v = *(const float4*)(src + i);
                alignas(16) T o[4] = {cast_to<T>(v.x), cast_to<T>(v.y), cast_to<T>(v.z), cast_to<T>(v.w)};
                if constexpr (sizeof(T) == 2) *(uint2*)(dst + i) = *(const uint2*)o;
                else *(float4*)(dst + i) = *(const float4*)o;
            } else {
                for (int64_t e = i; e < total && e < i + 4; ++e) dst[e] = cast_to<T>(src[e]);
            }
        }
        return;
    }
    const int tiles_c = (c + CAST_TILE - 1) / CAST_TILE, tiles_a = (a + CAST_TILE - 1) / CAST_TILE;
    const int tc = (int)(local % tiles_c);
    const int ta = (int)((local / tiles_c) % tiles_a);
    const int tap = (int)(local / ((int64_t)tiles_c * tiles_a));
    const int a0 = ta * CAST_TILE, c0 = tc * CAST_TILE;
    const int lane = tid & 63, r4 = tid >> 6;
    for (int r = r4; r < CAST_TILE; r += 4) {
        const int row = a0 + r, col = c0 + lane;
        tile[r][lane] = (row < a && col < c) ? src[((int64_t)row * b + tap) * c + col] : 0.f;
    }
    __syncthreads();
    for (int r = r4; r < CAST_TILE; r += 4) {
        const int crow = c0 + r, acol = a0 + lane;
        if (crow < c && acol < a) dst[((int64_t)crow * b + (b - 1 - tap)) * a + acol] = cast_to<T>(tile[lane][r]);
    }
}

}  // namespace

extern "C" int64_t ptv3_cast_params_blocks(int a, int b, int c, int mirror) {
    if (a <= 0 || b <= 0 || c <= 0) return 0;
    if (!mirror) return ptv3_ceil_div((int64_t)a * b * c, CAST_CHUNK);
    return (int64_t)b * ptv3_ceil_div(a, CAST_TILE) * ptv3_ceil_div(c, CAST_TILE);
}

extern "C" int ptv3_cast_params(const ptv3_cast_job* jobs, int n_jobs, int64_t n_blocks, int dst_dtype,
                                void* stream) {
    if (n_jobs < 0 || n_blocks < 0 || n_blocks > 0x7fffffffLL) return PTV3_EINVAL;
    if (n_jobs == 0 || n_blocks == 0) return PTV3_OK;
    if (!jobs) return PTV3_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)n_blocks), block(256);
    switch (dst_dtype) {
        case PTV3_F32: hipLaunchKernelGGL(cast_params_kernel<float>, grid, block, 0, s, jobs, n_jobs); break;
        case PTV3_F16: hipLaunchKernelGGL(cast_params_kernel<__half>, grid, block, 0, s, jobs, n_jobs); break;
        case PTV3_BF16: hipLaunchKernelGGL(cast_params_kernel<__hip_bfloat16>, grid, block, 0, s, jobs, n_jobs); break;
        default: return PTV3_EINVAL;
    }
    PTV3_RETURN_LAUNCH();
}
