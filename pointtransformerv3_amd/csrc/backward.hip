// Backward kernels of the sparse operators around the attention: the weight gradient of the
// submanifold convolution and the gradient of the segment reductions of grid pooling.
//
// * spconv.SubMConv3d (call sites model.py:546-552, :767-774): for out[i] = sum_t W[:,t,:] x[nbr[i][t]]
//   the input gradient is the same convolution with the taps mirrored and the weight transposed
//   (nbr[i][t] = j  <=>  nbr[j][V-1-t] = i), which the forward kernels already compute; what is new
//   is   dW[co][t][ci] = sum_i dy[i][co] * x[nbr[i][t]][ci],   here per (tap, 64x64 weight block, range of
//   voxels): both operands go through LDS 32 voxels at a time, every thread keeps a 4x4 block of sums
//   in fp32 and adds it to the fp32 result with atomics at the end.
// * torch_scatter.segment_csr (model.py:684-689): max / min send the gradient of a cluster to the first
//   member that attains the value, sum copies it to every member, mean divides it by the cluster size.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

constexpr int WG_T = 64;     // weight block: WG_T output x WG_T input channels
constexpr int WG_P = 32;     // voxels per staging step

template <typename T>
__global__ __launch_bounds__(256) void conv_wgrad_kernel(const T* __restrict__ x, const T* __restrict__ dy, int64_t n,
                                                         int cin, int cout, const int32_t* __restrict__ nbr, int taps,
                                                         int splits, int64_t rows_per_split, float* __restrict__ dw) {
    __shared__ float ys[WG_P][WG_T + 4];
    __shared__ float xs[WG_P][WG_T + 4];
    const int tap = blockIdx.x / splits, split = blockIdx.x % splits;
    const int co0 = blockIdx.y * WG_T, ci0 = blockIdx.z * WG_T;
    const int tid = threadIdx.x;
    const int ty = tid / 16, tx = tid % 16;
    const int64_t r0 = (int64_t)split * rows_per_split;
    const int64_t r1 = min(n, r0 + rows_per_split);
    const int32_t* nb = nbr + (int64_t)tap * n;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    const int c = tid % WG_T, p_of = tid / WG_T;   // staging: 4 voxels per pass of the work-group, 8 passes
    for (int64_t base = r0; base < r1; base += WG_P) {
        int32_t src[WG_P / 4];
        bool any = false;
#pragma unroll
        for (int k = 0; k < WG_P / 4; ++k) {
            const int64_t i = base + p_of + 4 * k;
            src[k] = i < r1 ? nb[i] : -1;
            any |= src[k] >= 0;
        }
        if (!__syncthreads_or(any)) continue;   // none of these voxels has this neighbour
#pragma unroll
        for (int k = 0; k < WG_P / 4; ++k) {
            const int p = p_of + 4 * k;
            const int64_t i = base + p;
            float yv = 0.f, xv = 0.f;
            if (src[k] >= 0) {
                if (co0 + c < cout) yv = (float)dy[i * cout + co0 + c];
                if (ci0 + c < cin) xv = (float)x[(int64_t)src[k] * cin + ci0 + c];
            }
            ys[p][c] = yv;
            xs[p][c] = xv;
        }
        __syncthreads();
#pragma unroll 8
        for (int p = 0; p < WG_P; ++p) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = ys[p][ty * 4 + i];
                b[i] = xs[p][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int co = co0 + ty * 4 + i, ci = ci0 + tx * 4 + j;
            if (co < cout && ci < cin && acc[i][j] != 0.f)
                atomicAdd(dw + ((int64_t)co * taps + tap) * cin + ci, acc[i][j]);
        }
}

// one thread per (cluster, channel): walks the members in list order
template <typename T>
__global__ __launch_bounds__(256) void segment_reduce_bwd_kernel(const T* __restrict__ src, const T* __restrict__ out,
                                                                 const T* __restrict__ dout, int c,
                                                                 const int64_t* __restrict__ indices,
                                                                 const int64_t* __restrict__ idx_ptr, int64_t m, int op,
                                                                 T* __restrict__ dsrc) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= m * c) return;
    const int64_t s = e / c;
    const int ch = (int)(e - s * c);
    const int64_t b = idx_ptr[s], t = idx_ptr[s + 1];
    const float g = (float)dout[e];
    if (op == 0 || op == 3) {
        const T best = out[e];
        bool taken = false;
        for (int64_t j = b; j < t; ++j) {
            const int64_t row = indices[j];
            const bool hit = !taken && (float)src[row * c + ch] == (float)best;
            taken |= hit;
            dsrc[row * c + ch] = hit ? (T)g : (T)0.f;
        }
    } else {
        const T v = (T)(op == 1 ? g / (float)(t - b) : g);
        for (int64_t j = b; j < t; ++j) dsrc[indices[j] * c + ch] = v;
    }
}

template <typename T>
int launch_wgrad(const void* x, const void* dy, int64_t n, int cin, int cout, const int32_t* nbr, int taps, float* dw,
                 hipStream_t stream) {
    const int ct = (int)(ptv3_ceil_div(cout, WG_T) * ptv3_ceil_div(cin, WG_T));
    // enough work-groups to fill the part several times, at least 256 voxels each
    int64_t splits = ptv3_ceil_div(8192, (int64_t)taps * ct);
    const int64_t most = ptv3_ceil_div(n, 256);
    if (splits > most) splits = most;
    if (splits < 1) splits = 1;
    const int64_t rows = ptv3_ceil_div(ptv3_ceil_div(n, splits), WG_P) * WG_P;
    splits = ptv3_ceil_div(n, rows);
    hipLaunchKernelGGL(conv_wgrad_kernel<T>, dim3((unsigned)(taps * splits), (unsigned)ptv3_ceil_div(cout, WG_T),
                                                  (unsigned)ptv3_ceil_div(cin, WG_T)),
                       dim3(256), 0, stream, (const T*)x, (const T*)dy, n, cin, cout, nbr, taps, (int)splits, rows, dw);
    PTV3_RETURN_LAUNCH();
}

template <typename T>
int launch_segment_bwd(const void* src, const void* out, const void* dout, int c, const int64_t* indices,
                       const int64_t* idx_ptr, int64_t m, int op, void* dsrc, hipStream_t stream) {
    hipLaunchKernelGGL(segment_reduce_bwd_kernel<T>, dim3((unsigned)ptv3_ceil_div(m * c, 256)), dim3(256), 0, stream,
                       (const T*)src, (const T*)out, (const T*)dout, c, indices, idx_ptr, m, op, (T*)dsrc);
    PTV3_RETURN_LAUNCH();
}

}  // namespace

extern "C" int ptv3_subm_conv_wgrad(const void* feat, const void* dout, int dtype, int64_t n, int cin, int cout,
                                    const int32_t* nbr, int taps, float* dweight, void* stream_) {
    if (n < 0 || cin < 1 || cout < 1 || taps < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!feat || !dout || !nbr || !dweight) return PTV3_EINVAL;
    if ((int64_t)taps * ptv3_ceil_div(n, 256) >= (1ll << 31)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16) return launch_wgrad<_Float16>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
    if (dtype == PTV3_BF16) return launch_wgrad<__bf16>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
    return launch_wgrad<float>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
}

extern "C" int ptv3_segment_reduce_bwd(const void* src, const void* out, const void* dout, int dtype, int64_t n, int c,
                                       const int64_t* indices, const int64_t* idx_ptr, int64_t m, int op, void* dsrc,
                                       void* stream_) {
    if (n < 0 || m < 0 || c < 1 || op < 0 || op > 3) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (m == 0 || n == 0) return PTV3_OK;
    if (!src || !out || !dout || !indices || !idx_ptr || !dsrc) return PTV3_EINVAL;
    if (ptv3_ceil_div(m * c, 256) >= (1ll << 31)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16)
        return launch_segment_bwd<_Float16>(src, out, dout, c, indices, idx_ptr, m, op, dsrc, stream);
    if (dtype == PTV3_BF16)
        return launch_segment_bwd<__bf16>(src, out, dout, c, indices, idx_ptr, m, op, dsrc, stream);
    return launch_segment_bwd<float>(src, out, dout, c, indices, idx_ptr, m, op, dsrc, stream);
}
