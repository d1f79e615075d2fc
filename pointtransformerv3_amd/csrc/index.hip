// Patch padding tables and the per-order gather/scatter tables of serialized attention.
//
// Replaces model.py:392-437 (a Python loop over scenes with one device->host sync per
// scene in the reference) and the index arithmetic of model.py:452-453 by two launches
// that never leave the device.
#include "common.h"

namespace {

// Single thread: exclusive prefix of padded scene lengths and of sequence counts.
__global__ void pad_prefix_kernel(const int64_t* __restrict__ offset, int nb, int64_t patch,
                                  int64_t* __restrict__ pad_start, int64_t* __restrict__ seq_start) {
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    int64_t prev = 0, op = 0, sq = 0;
    for (int s = 0; s < nb; ++s) {
        const int64_t cnt = offset[s] - prev;
        prev = offset[s];
        const int64_t padded = cnt > patch ? ((cnt + patch - 1) / patch) * patch : cnt;
        pad_start[s] = op;
        seq_start[s] = sq;
        op += padded;
        sq += (padded + patch - 1) / patch;
    }
    pad_start[nb] = op;
    seq_start[nb] = sq;
}

__global__ __launch_bounds__(256) void pad_index_kernel(
    const int64_t* __restrict__ offset, int nb, int64_t patch, int64_t n_pad, int64_t n_seq,
    const int64_t* __restrict__ pad_start, const int64_t* __restrict__ seq_start,
    int64_t* __restrict__ pad, int64_t* __restrict__ unpad, int32_t* __restrict__ cu_seqlens) {
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j == 0) cu_seqlens[n_seq] = (int32_t)n_pad;
    if (j >= n_pad) return;
    // scene s: last s with pad_start[s] <= j (empty scenes share a start and are skipped)
    int lo = 0, hi = nb;  // invariant: pad_start[lo] <= j < pad_start[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (pad_start[mid] <= j) lo = mid; else hi = mid;
    }
    const int s = lo;
    const int64_t first = s ? offset[s - 1] : 0;
    const int64_t cnt = offset[s] - first;
    const int64_t local = j - pad_start[s];
    // filler slots of the last patch reuse the points one patch earlier (model.py:412-423)
    pad[j] = first + (local < cnt ? local : local - patch);
    if (local < cnt) unpad[first + local] = j;
    if (local % patch == 0) cu_seqlens[seq_start[s] + local / patch] = (int32_t)j;
}

__global__ __launch_bounds__(256) void attn_slots_kernel(
    const int64_t* __restrict__ order_row, const int64_t* __restrict__ inverse_row,
    const int64_t* __restrict__ pad, const int64_t* __restrict__ unpad, int64_t n_pad,
    int32_t* __restrict__ slot_src, int32_t* __restrict__ slot_dst) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_pad) return;
    const int64_t row = order_row[pad[i]];
    slot_src[i] = (int32_t)row;
    slot_dst[i] = (unpad[inverse_row[row]] == i) ? (int32_t)row : -1;
}

// per-axis maximum of (n,3) int32 coordinates into out[3] (pre-set to INT_MIN by the caller's
// first kernel below): wave and block reduce, then one atomic per block and axis
__global__ void grid_max_init_kernel(int32_t* __restrict__ out) {
    if (threadIdx.x < 3) out[threadIdx.x] = INT32_MIN;
}

__global__ __launch_bounds__(256) void grid_max_kernel(const int32_t* __restrict__ grid_coord, int64_t n,
                                                       int head, int32_t* __restrict__ out) {
    // the (n,3) array as a flat stream of 3n values, value f being axis f % 3: `head` values up to
    // the first 16-byte boundary, then four per load, then the last few
    typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
    __shared__ int32_t part[4][3];
    int32_t m[3] = {INT32_MIN, INT32_MIN, INT32_MIN};
    const int64_t total = 3 * n, quads = (total - head) / 4;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        const i32x4 v = *(const i32x4*)(grid_coord + head + 4 * q);
        const int a0 = (int)((head + 4 * q) % 3);   // axis of v[0] and v[3]; v[1], v[2] follow cyclically
        const int a1 = a0 == 2 ? 0 : a0 + 1;
        const int32_t first = max(v[0], v[3]);
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const int32_t c = a == a0 ? first : (a == a1 ? v[1] : v[2]);
            m[a] = max(m[a], c);
        }
    }
    if (blockIdx.x == 0) {   // at most 3 + 3 leftover values
        const int64_t rest = total - head - 4 * quads;
        int64_t f = -1;
        if ((int)threadIdx.x < head) f = threadIdx.x;
        else if ((int64_t)threadIdx.x - head < rest) f = 4 * quads + threadIdx.x;
        if (f >= 0) {
            const int a = (int)(f % 3);
            const int32_t v = grid_coord[f];
#pragma unroll
            for (int k = 0; k < 3; ++k) if (k == a) m[k] = max(m[k], v);
        }
    }
    const int wave = threadIdx.x / PTV3_WAVE, lane = threadIdx.x % PTV3_WAVE;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m[a] = max(m[a], __shfl_xor(m[a], off, PTV3_WAVE));
        if (lane == 0) part[wave][a] = m[a];
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const int a = threadIdx.x;
        atomicMax(&out[a], max(max(part[0][a], part[1][a]), max(part[2][a], part[3][a])));
    }
}

// scene id of every point from the cumulative scene ends: the number of ends <= i
__global__ __launch_bounds__(256) void offset2batch_kernel(const int64_t* __restrict__ offset, int nb, int64_t n,
                                                           int64_t* __restrict__ batch) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    int lo = 0, hi = nb;   // first scene whose end is > i
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (offset[mid] <= i) lo = mid + 1; else hi = mid;
    }
    batch[i] = lo;
}

}  // namespace

extern "C" int ptv3_offset2batch(const int64_t* offset, int n_scenes, int64_t n, int64_t* batch, void* stream_) {
    if (n < 0 || n_scenes < 1) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!offset || !batch) return PTV3_EINVAL;
    hipLaunchKernelGGL(offset2batch_kernel, dim3((unsigned)ptv3_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream_,
                       offset, n_scenes, n, batch);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_grid_max(const int32_t* grid_coord, int64_t n, int32_t* out3, void* stream_) {
    if (n < 1 || !grid_coord || !out3) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    hipLaunchKernelGGL(grid_max_init_kernel, dim3(1), dim3(64), 0, stream, out3);
    const int64_t want = ptv3_ceil_div(3 * n, 4 * 256);   // one 16-byte load per thread, at most 512 blocks
    const int64_t blocks = want < 512 ? want : 512;
    int head = (int)(((16 - ((uintptr_t)grid_coord & 15)) & 15) / 4);
    if (head > 3 * n) head = (int)(3 * n);
    hipLaunchKernelGGL(grid_max_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, grid_coord, n, head, out3);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_pad_sizes(const int64_t* offset_host, int nb, int64_t patch, int64_t* n_pad,
                              int64_t* n_seq) {
    if (!offset_host || nb < 0 || patch < 1 || !n_pad || !n_seq) return PTV3_EINVAL;
    int64_t prev = 0, op = 0, sq = 0;
    for (int s = 0; s < nb; ++s) {
        const int64_t cnt = offset_host[s] - prev;
        if (cnt < 0) return PTV3_EINVAL;
        prev = offset_host[s];
        const int64_t padded = cnt > patch ? ((cnt + patch - 1) / patch) * patch : cnt;
        op += padded;
        sq += (padded + patch - 1) / patch;
    }
    *n_pad = op;
    *n_seq = sq;
    return PTV3_OK;
}

extern "C" size_t ptv3_pad_index_workspace_bytes(int nb) {
    return nb < 0 ? 0 : ptv3_align256(2 * (size_t)(nb + 1) * sizeof(int64_t));
}

extern "C" int ptv3_pad_index(const int64_t* offset, int nb, int64_t patch, int64_t n,
                              int64_t n_pad, int64_t n_seq, int64_t* pad, int64_t* unpad,
                              int32_t* cu_seqlens, void* workspace, size_t workspace_bytes,
                              void* stream_) {
    if (nb < 1 || patch < 1 || n < 0 || n_pad < n || n_seq < 0 || n_pad >= (1ll << 31))
        return PTV3_EINVAL;
    if (!offset || !cu_seqlens || !workspace) return PTV3_EINVAL;
    if (n_pad > 0 && (!pad || !unpad)) return PTV3_EINVAL;
    if (workspace_bytes < ptv3_pad_index_workspace_bytes(nb)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    int64_t* pad_start = (int64_t*)workspace;
    int64_t* seq_start = pad_start + (nb + 1);
    hipLaunchKernelGGL(pad_prefix_kernel, dim3(1), dim3(1), 0, stream, offset, nb, patch, pad_start,
                       seq_start);
    const int64_t blocks = ptv3_ceil_div(n_pad > 0 ? n_pad : 1, 256);
    hipLaunchKernelGGL(pad_index_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, offset, nb,
                       patch, n_pad, n_seq, (const int64_t*)pad_start, (const int64_t*)seq_start,
                       pad, unpad, cu_seqlens);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_attn_slots(const int64_t* order_row, const int64_t* inverse_row,
                               const int64_t* pad, const int64_t* unpad, int64_t n_pad,
                               int32_t* slot_src, int32_t* slot_dst, void* stream) {
    if (n_pad < 0 || n_pad >= (1ll << 31)) return PTV3_EINVAL;
    if (n_pad == 0) return PTV3_OK;
    if (!order_row || !inverse_row || !pad || !unpad || !slot_src || !slot_dst) return PTV3_EINVAL;
    const int64_t blocks = ptv3_ceil_div(n_pad, 256);
    hipLaunchKernelGGL(attn_slots_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       order_row, inverse_row, pad, unpad, n_pad, slot_src, slot_dst);
    PTV3_RETURN_LAUNCH();
}
