// Pair lists ("plan") for the sparse-pair form of the submanifold convolution.
//
// The reference's spconv builds, per kernel offset, the list of (input, output) index pairs
// that are active (call sites model.py:546-552, :767-774). This file derives the same pairs
// from the neighbour map in two orders at once:
//   * tap-major pair index q: all pairs of tap 0, then tap 1, ... (tap_ptr[taps+1]); inside a
//     tap, output voxels ascend. Rows of one GEMM tile share a tap and therefore a weight
//     matrix, so MFMA tiles are fully populated whatever the per-voxel sparsity is.
//   * output-major slot s: the pairs of voxel 0, then voxel 1, ... (row_ptr[n+1]); the GEMM
//     writes pair q's product row to y[pair_slot[q]], and a segment sum over
//     [row_ptr[i], row_ptr[i+1]) finishes voxel i without atomics.
// Both ranks are exclusive scans of the same activity mask, one row-major, one tap-major.
#include "common.h"

namespace {

constexpr int PLAN_THREADS = 256;
constexpr int PLAN_WAVES = PLAN_THREADS / PTV3_WAVE;
constexpr int MAX_TAPS = 128;

__device__ __forceinline__ uint32_t block_scan_incl(uint32_t v, uint32_t* total) {
    __shared__ uint32_t wsum[PLAN_WAVES];
    const int lane = threadIdx.x % PTV3_WAVE, wave = threadIdx.x / PTV3_WAVE;
    uint32_t x = v;
#pragma unroll
    for (int off = 1; off < PTV3_WAVE; off <<= 1) {
        const uint32_t y = __shfl_up(x, off, PTV3_WAVE);
        if (lane >= off) x += y;
    }
    if (lane == PTV3_WAVE - 1) wsum[wave] = x;
    __syncthreads();
    uint32_t base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < PLAN_WAVES; ++w) {
        const uint32_t c = wsum[w];
        if (w < wave) base += c;
        tot += c;
    }
    *total = tot;
    __syncthreads();
    return x + base;
}

// thread = voxel: active taps of the voxel, and active voxels of the block per tap
// entry (voxel i, tap t) of a map stored voxel-major (n,taps) or tap-major (taps,n)
__device__ __forceinline__ int32_t nbr_at(const int32_t* __restrict__ nbr, int64_t n, int taps, bool tap_major,
                                          int64_t i, int t) {
    return tap_major ? nbr[(int64_t)t * n + i] : nbr[i * taps + t];
}

__global__ __launch_bounds__(PLAN_THREADS) void plan_count_kernel(
    const int32_t* __restrict__ nbr, int64_t n, int taps, bool tap_major, uint32_t* __restrict__ row_cnt,
    uint32_t* __restrict__ blk_row_sum, uint32_t* __restrict__ blk_tap_cnt) {
    __shared__ uint32_t tapcnt[MAX_TAPS];
    const int tid = threadIdx.x, lane = tid % PTV3_WAVE;
    const int64_t i = (int64_t)blockIdx.x * PLAN_THREADS + tid;
    if (tid < MAX_TAPS) tapcnt[tid] = 0;
    __syncthreads();
    uint32_t cnt = 0;
    for (int t = 0; t < taps; ++t) {
        const bool a = i < n && nbr_at(nbr, n, taps, tap_major, i, t) >= 0;
        cnt += a;
        const uint64_t bal = __ballot(a);
        if (lane == 0 && bal) atomicAdd(&tapcnt[t], (uint32_t)__popcll(bal));
    }
    if (i < n) row_cnt[i] = cnt;
    uint32_t total;
    block_scan_incl(cnt, &total);
    if (tid == 0) blk_row_sum[blockIdx.x] = total;
    __syncthreads();
    if (tid < taps) blk_tap_cnt[(int64_t)blockIdx.x * taps + tid] = tapcnt[tid];
}

// blockIdx.x < taps: exclusive scan of column t of blk_tap_cnt over the blocks, total to
// tap_total[t]. blockIdx.x == taps: exclusive scan of blk_row_sum, grand total to *n_pairs.
__global__ __launch_bounds__(PLAN_THREADS) void plan_scan_kernel(uint32_t* __restrict__ blk_tap_cnt,
                                                                 uint32_t* __restrict__ blk_row_sum,
                                                                 int64_t blocks, int taps,
                                                                 uint32_t* __restrict__ tap_total,
                                                                 int64_t* __restrict__ n_pairs) {
    const int col = blockIdx.x;
    uint32_t carry = 0;
    for (int64_t b0 = 0; b0 < blocks; b0 += PLAN_THREADS) {
        const int64_t b = b0 + threadIdx.x;
        uint32_t* p = col < taps ? &blk_tap_cnt[b * taps + col] : &blk_row_sum[b];
        const uint32_t v = b < blocks ? *p : 0u;
        uint32_t total;
        const uint32_t inc = block_scan_incl(v, &total);
        if (b < blocks) *p = carry + inc - v;
        carry += total;
    }
    if (threadIdx.x == 0) {
        if (col < taps) tap_total[col] = carry;
        else *n_pairs = (int64_t)carry;
    }
}

// single block: tap_ptr = exclusive scan of tap_total (taps <= 128)
__global__ __launch_bounds__(PLAN_THREADS) void plan_tap_ptr_kernel(const uint32_t* __restrict__ tap_total,
                                                                    int taps, int32_t* __restrict__ tap_ptr) {
    const int t = threadIdx.x;
    const uint32_t v = t < taps ? tap_total[t] : 0u;
    uint32_t total;
    const uint32_t inc = block_scan_incl(v, &total);
    if (t < taps) tap_ptr[t] = (int32_t)(inc - v);
    if (t == 0) tap_ptr[taps] = (int32_t)total;
}

// thread = voxel: row_ptr, and for every active (voxel, tap) the pair entry
__global__ __launch_bounds__(PLAN_THREADS) void plan_fill_kernel(
    const int32_t* __restrict__ nbr, int64_t n, int taps, bool tap_major, const uint32_t* __restrict__ row_cnt,
    const uint32_t* __restrict__ blk_row_off, const uint32_t* __restrict__ blk_tap_off,
    const int32_t* __restrict__ tap_ptr, int32_t* __restrict__ row_ptr, int32_t* __restrict__ pair_in,
    int32_t* __restrict__ pair_slot) {
    __shared__ uint32_t wave_tap[PLAN_WAVES][MAX_TAPS];
    const int tid = threadIdx.x, lane = tid % PTV3_WAVE, wave = tid / PTV3_WAVE;
    const int64_t i = (int64_t)blockIdx.x * PLAN_THREADS + tid;
    const uint64_t below = (1ull << lane) - 1ull;
    // per-wave, per-tap activity counts
    for (int t = 0; t < taps; ++t) {
        const bool a = i < n && nbr_at(nbr, n, taps, tap_major, i, t) >= 0;
        const uint64_t bal = __ballot(a);
        if (lane == 0) wave_tap[wave][t] = (uint32_t)__popcll(bal);
    }
    // first output slot of my voxel
    const uint32_t cnt = i < n ? row_cnt[i] : 0u;
    uint32_t total;
    const uint32_t inc = block_scan_incl(cnt, &total);   // also orders the wave_tap writes
    uint32_t slot = blk_row_off[blockIdx.x] + inc - cnt;
    if (i < n) row_ptr[i] = (int32_t)slot;
    if (i == n - 1) row_ptr[n] = (int32_t)(slot + cnt);
    for (int t = 0; t < taps; ++t) {
        const int32_t src = i < n ? nbr_at(nbr, n, taps, tap_major, i, t) : -1;
        const bool a = src >= 0;
        const uint64_t bal = __ballot(a);
        if (a) {
            uint32_t q = (uint32_t)tap_ptr[t] + blk_tap_off[(int64_t)blockIdx.x * taps + t] +
                         (uint32_t)__popcll(bal & below);
            for (int w = 0; w < wave; ++w) q += wave_tap[w][t];
            pair_in[q] = src;
            pair_slot[q] = (int32_t)slot;
            ++slot;
        }
    }
}

struct PlanWs {
    uint32_t *row_cnt, *blk_row_sum, *blk_tap_cnt, *tap_total;
    size_t bytes;
};

PlanWs carve_plan(void* base, int64_t n, int taps) {
    const int64_t blocks = ptv3_ceil_div(n > 0 ? n : 1, PLAN_THREADS);
    PlanWs w;
    char* p = (char*)base;
    size_t off = 0;
    w.row_cnt = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)(n > 0 ? n : 1) * 4);
    w.blk_row_sum = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)blocks * 4);
    w.blk_tap_cnt = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)blocks * taps * 4);
    w.tap_total = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)MAX_TAPS * 4);
    w.bytes = off;
    return w;
}

}  // namespace

extern "C" size_t ptv3_conv_plan_workspace_bytes(int64_t n, int taps) {
    if (n < 0 || taps < 1 || taps > MAX_TAPS) return 0;
    return carve_plan(nullptr, n, taps).bytes;
}

extern "C" int ptv3_conv_plan_count(const int32_t* nbr, int64_t n, int taps, int tap_major, int32_t* tap_ptr,
                                    int64_t* n_pairs, void* workspace, size_t workspace_bytes,
                                    void* stream_) {
    if (n < 1 || n >= (1ll << 31) / 128 || taps < 1 || taps > MAX_TAPS) return PTV3_EINVAL;
    if (!nbr || !tap_ptr || !n_pairs || !workspace) return PTV3_EINVAL;
    PlanWs w = carve_plan(workspace, n, taps);
    if (workspace_bytes < w.bytes) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const int64_t blocks = ptv3_ceil_div(n, PLAN_THREADS);
    hipLaunchKernelGGL(plan_count_kernel, dim3((unsigned)blocks), dim3(PLAN_THREADS), 0, stream, nbr, n, taps,
                       tap_major != 0, w.row_cnt, w.blk_row_sum, w.blk_tap_cnt);
    hipLaunchKernelGGL(plan_scan_kernel, dim3((unsigned)(taps + 1)), dim3(PLAN_THREADS), 0, stream,
                       w.blk_tap_cnt, w.blk_row_sum, blocks, taps, w.tap_total, n_pairs);
    hipLaunchKernelGGL(plan_tap_ptr_kernel, dim3(1), dim3(PLAN_THREADS), 0, stream,
                       (const uint32_t*)w.tap_total, taps, tap_ptr);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_conv_plan_fill(const int32_t* nbr, int64_t n, int taps, int tap_major, const int32_t* tap_ptr,
                                   int32_t* row_ptr, int32_t* pair_in, int32_t* pair_slot,
                                   void* workspace, size_t workspace_bytes, void* stream_) {
    if (n < 1 || n >= (1ll << 31) / 128 || taps < 1 || taps > MAX_TAPS) return PTV3_EINVAL;
    if (!nbr || !tap_ptr || !row_ptr || !pair_in || !pair_slot || !workspace) return PTV3_EINVAL;
    PlanWs w = carve_plan(workspace, n, taps);
    if (workspace_bytes < w.bytes) return PTV3_EWORKSPACE;
    const int64_t blocks = ptv3_ceil_div(n, PLAN_THREADS);
    hipLaunchKernelGGL(plan_fill_kernel, dim3((unsigned)blocks), dim3(PLAN_THREADS), 0, (hipStream_t)stream_,
                       nbr, n, taps, tap_major != 0, (const uint32_t*)w.row_cnt, (const uint32_t*)w.blk_row_sum,
                       (const uint32_t*)w.blk_tap_cnt, tap_ptr, row_ptr, pair_in, pair_slot);
    PTV3_RETURN_LAUNCH();
}
