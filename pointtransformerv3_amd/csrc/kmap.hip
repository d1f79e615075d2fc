// Submanifold neighbour map ("kmap") through an open-addressing voxel hash.
//
// Replaces the index generation spconv performs for SubMConv3d (reference call sites
// model.py:546-552 and :767-774 on the tensor built at :165-172). Canonical output:
// entry (voxel i, tap (kx*ks+ky)*ks+kz) = row of the voxel at coord_i + (kx,ky,kz) - ks/2, or -1,
// stored voxel-major (n, taps) or tap-major (taps, n); the convolution kernels read the
// tap-major form coalesced.
//
//   fill, insert : the block-keyed voxel hash (voxelhash.h)
//   lookup       : one thread per voxel: at most 8 block headers tell which neighbours exist, one row
//                  read per existing neighbour; the voxel's taps are first set to -1 (in the
//                  tap-major layout consecutive lanes write consecutive voxels of one tap).
#include "voxelhash.h"

namespace {

template <bool TAP_MAJOR, int KS>
__global__ __launch_bounds__(256) void kmap_lookup_kernel(const int32_t* __restrict__ indices, int64_t n,
                                                          VoxelHash h, int32_t* __restrict__ nbr) {
    constexpr int R = KS / 2, TAPS = KS * KS * KS;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 v = ((const int4*)indices)[i];
    const VoxelWindow w = vh_window<R>(h, v.x, v.y, v.z, v.w);
#pragma unroll 1
    for (int t = 0; t < TAPS; ++t) nbr[TAP_MAJOR ? (int64_t)t * n + i : i * TAPS + t] = -1;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        uint64_t m = w.hits[k];
        while (m) {
            const int bit = __builtin_ctzll(m);
            m &= m - 1;
            const int t = vh_tap_of<R>(w, k, bit, v.y, v.z, v.w);
            const int32_t row = t == TAPS / 2 ? (int32_t)i : h.rows[(int64_t)w.slot[k] * 64 + bit];
            nbr[TAP_MAJOR ? (int64_t)t * n + i : i * TAPS + t] = row;
        }
    }
}

}  // namespace

extern "C" size_t ptv3_kmap_workspace_bytes(int64_t n) {
    if (n < 0) return 0;
    return vh_bytes(n);
}

extern "C" int ptv3_kmap_build(const int32_t* indices, int64_t n, int ks, int tap_major, int32_t* nbr,
                               void* workspace, size_t workspace_bytes, void* stream_) {
    if (n < 0 || n >= (1ll << 30)) return PTV3_EINVAL;
    if (ks != 3 && ks != 5) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!indices || !nbr || !workspace) return PTV3_EINVAL;
    if (workspace_bytes < vh_bytes(n)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const VoxelHash h = vh_build(workspace, indices, n, stream);
    const dim3 grid((unsigned)ptv3_ceil_div(n, 256)), block(256);
#define PTV3_LOOKUP(TM, KS) hipLaunchKernelGGL((kmap_lookup_kernel<TM, KS>), grid, block, 0, stream, indices, n, h, nbr)
    if (tap_major) {
        if (ks == 3) PTV3_LOOKUP(true, 3); else PTV3_LOOKUP(true, 5);
    } else {
        if (ks == 3) PTV3_LOOKUP(false, 3); else PTV3_LOOKUP(false, 5);
    }
#undef PTV3_LOOKUP
    PTV3_RETURN_LAUNCH();
}
