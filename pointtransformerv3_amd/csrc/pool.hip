// Grid pooling / unpooling as segment operations over the serialized order.
//
// Replaces model.py:652-664 (torch.unique + torch.sort + cumsum), :666,:690,:695 (head
// gathers), :684-689 (torch_scatter.segment_csr) and :746 (gather-add) of the reference.
// The points are already sorted by row-0 code, so clusters of `code0 >> shift` are runs in
// that order: boundary flags + an exclusive scan number them; no sort, no hash.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <mutex>

#include "common.h"

namespace {

constexpr int PB = 256;   // threads per block in the scan kernels

__device__ __forceinline__ bool run_start(const int64_t* __restrict__ code0,
                                          const int64_t* __restrict__ order0, int64_t i, int shift) {
    if (i == 0) return true;
    return (code0[order0[i]] >> shift) != (code0[order0[i - 1]] >> shift);
}

// inclusive scan of one value per thread across a 256-thread block; returns the inclusive
// prefix and leaves the block total in *total.
__device__ __forceinline__ uint32_t block_inclusive_scan(uint32_t v, uint32_t* total) {
    __shared__ uint32_t wsum[PB / PTV3_WAVE];
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
    for (int w = 0; w < PB / PTV3_WAVE; ++w) {
        const uint32_t c = wsum[w];
        if (w < wave) base += c;
        tot += c;
    }
    *total = tot;
    __syncthreads();
    return x + base;
}

__global__ __launch_bounds__(PB) void cluster_count_kernel(const int64_t* __restrict__ code0,
                                                           const int64_t* __restrict__ order0,
                                                           int64_t n, int shift,
                                                           uint32_t* __restrict__ block_cnt) {
    const int64_t i = (int64_t)blockIdx.x * PB + threadIdx.x;
    const uint32_t f = (i < n && run_start(code0, order0, i, shift)) ? 1u : 0u;
    uint32_t total;
    block_inclusive_scan(f, &total);
    if (threadIdx.x == 0) block_cnt[blockIdx.x] = total;
}

// single block: exclusive scan of block_cnt in place, grand total to n_clusters
__global__ __launch_bounds__(PB) void cluster_scan_kernel(uint32_t* __restrict__ block_cnt,
                                                          int64_t blocks,
                                                          int64_t* __restrict__ n_clusters) {
    uint32_t carry = 0;
    for (int64_t b0 = 0; b0 < blocks; b0 += PB) {
        const int64_t b = b0 + threadIdx.x;
        const uint32_t v = b < blocks ? block_cnt[b] : 0u;
        uint32_t total;
        const uint32_t inc = block_inclusive_scan(v, &total);
        if (b < blocks) block_cnt[b] = carry + inc - v;
        carry += total;
    }
    if (threadIdx.x == 0) *n_clusters = (int64_t)carry;
}

__global__ __launch_bounds__(PB) void cluster_assign_kernel(
    const int64_t* __restrict__ code0, const int64_t* __restrict__ order0, int64_t n, int shift,
    const uint32_t* __restrict__ block_base, int64_t* __restrict__ cluster,
    int64_t* __restrict__ idx_ptr, int64_t* __restrict__ head) {
    const int64_t i = (int64_t)blockIdx.x * PB + threadIdx.x;
    const bool f = i < n && run_start(code0, order0, i, shift);
    uint32_t total;
    const uint32_t inc = block_inclusive_scan(f ? 1u : 0u, &total);
    if (i >= n) return;
    const int64_t cid = (int64_t)block_base[blockIdx.x] + inc - 1;
    const int64_t pt = order0[i];
    cluster[pt] = cid;
    if (f) {
        idx_ptr[cid] = i;
        head[cid] = pt;
    }
    if (i == n - 1) idx_ptr[cid + 1] = n;
}

// ---- pooled serialization orders without sorting.
// Walking the parent points along any of their serialization orders visits the clusters of the
// coarser level as runs (a point's code shifted right by 3 bits per pooled level is its cluster's
// code on the same curve), in ascending order of that cluster code. The sequence of run heads is
// therefore the pooled order of that curve: flags + scan per row, all rows in one launch.
__device__ __forceinline__ bool order_run_start(const int64_t* __restrict__ order_row,
                                                const int64_t* __restrict__ cluster, int64_t i) {
    if (i == 0) return true;
    return cluster[order_row[i]] != cluster[order_row[i - 1]];
}

// Output row r of the pooled tables comes from input row src[r] (the reference permutes the rows
// after pooling, model.py:675-679: the same tables, written once).
constexpr int MAX_PERM_ROWS = 16;
struct RowPerm {
    int32_t src[MAX_PERM_ROWS];
    int use;
    __device__ __forceinline__ int of(int r) const { return use ? src[r] : r; }
};

RowPerm make_row_perm(const int32_t* host_perm, int k) {
    RowPerm p;
    p.use = host_perm != nullptr;
    for (int r = 0; r < MAX_PERM_ROWS; ++r) p.src[r] = (host_perm && r < k) ? host_perm[r] : r;
    return p;
}

bool row_perm_ok(const int32_t* host_perm, int k) {
    if (!host_perm) return true;
    if (k > MAX_PERM_ROWS) return false;
    for (int r = 0; r < k; ++r)
        if (host_perm[r] < 0 || host_perm[r] >= k) return false;
    return true;
}

__global__ __launch_bounds__(PB) void order_count_kernel(const int64_t* __restrict__ order,
                                                         const int64_t* __restrict__ cluster, int64_t n,
                                                         RowPerm perm, uint32_t* __restrict__ block_cnt) {
    const int64_t i = (int64_t)blockIdx.x * PB + threadIdx.x;
    const int64_t* row = order + (int64_t)perm.of(blockIdx.y) * n;
    const uint32_t f = (i < n && order_run_start(row, cluster, i)) ? 1u : 0u;
    uint32_t total;
    block_inclusive_scan(f, &total);
    if (threadIdx.x == 0) block_cnt[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = total;
}

// one block per row: exclusive scan of the row's block counts in place
__global__ __launch_bounds__(PB) void order_scan_kernel(uint32_t* __restrict__ block_cnt, int64_t blocks) {
    uint32_t* cnt = block_cnt + (int64_t)blockIdx.x * blocks;
    uint32_t carry = 0;
    for (int64_t b0 = 0; b0 < blocks; b0 += PB) {
        const int64_t b = b0 + threadIdx.x;
        const uint32_t v = b < blocks ? cnt[b] : 0u;
        uint32_t total;
        const uint32_t inc = block_inclusive_scan(v, &total);
        if (b < blocks) cnt[b] = carry + inc - v;
        carry += total;
    }
}

__global__ __launch_bounds__(PB) void order_assign_kernel(const int64_t* __restrict__ order,
                                                          const int64_t* __restrict__ cluster, int64_t n,
                                                          int64_t m, RowPerm perm,
                                                          const uint32_t* __restrict__ block_base,
                                                          int64_t* __restrict__ order_out,
                                                          int64_t* __restrict__ inverse_out) {
    const int64_t i = (int64_t)blockIdx.x * PB + threadIdx.x;
    const int64_t* row = order + (int64_t)perm.of(blockIdx.y) * n;
    const bool f = i < n && order_run_start(row, cluster, i);
    uint32_t total;
    const uint32_t inc = block_inclusive_scan(f ? 1u : 0u, &total);
    if (!f) return;
    const int64_t pos = (int64_t)block_base[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] + inc - 1;
    if (pos >= m) return;   // cannot happen when the codes form a hierarchy; keeps writes in bounds
    const int64_t c = cluster[row[i]];
    order_out[(int64_t)blockIdx.y * m + pos] = c;
    inverse_out[(int64_t)blockIdx.y * m + c] = pos;
}

__global__ __launch_bounds__(256) void pool_gather_kernel(
    const int64_t* __restrict__ code, int64_t n, int k, int shift,
    const int32_t* __restrict__ grid_coord, int pool_depth, const int64_t* __restrict__ batch,
    const int64_t* __restrict__ head, int64_t m, RowPerm perm, int64_t* __restrict__ code_out,
    int32_t* __restrict__ grid_coord_out, int64_t* __restrict__ batch_out, int32_t* __restrict__ indices_out) {
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= m) return;
    const int64_t h = head[j];
    for (int r = 0; r < k; ++r) code_out[(int64_t)r * m + j] = code[(int64_t)perm.of(r) * n + h] >> shift;
    int32_t g[3] = {0, 0, 0};
    if (grid_coord) {
#pragma unroll
        for (int a = 0; a < 3; ++a) g[a] = grid_coord[3 * h + a] >> pool_depth;
    }
    const int64_t b = batch ? batch[h] : 0;
    if (grid_coord_out) {
#pragma unroll
        for (int a = 0; a < 3; ++a) grid_coord_out[3 * j + a] = g[a];
    }
    if (batch_out) batch_out[j] = b;
    if (indices_out) ((int4*)indices_out)[j] = make_int4((int32_t)b, g[0], g[1], g[2]);
}

// pooled scene ends: scene s ends with the cluster of its last point in sorted order
__global__ __launch_bounds__(256) void pool_offsets_kernel(const int64_t* __restrict__ offset, int nb,
                                                           const int64_t* __restrict__ order0,
                                                           const int64_t* __restrict__ cluster,
                                                           int64_t* __restrict__ out) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= nb) return;
    const int64_t last = offset[j] - 1;   // -1: no point so far
    out[j] = last >= 0 ? cluster[order0[last]] + 1 : 0;
}

template <typename T> __device__ __forceinline__ float ld(const T* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void st(T* p, float v) { *p = (T)v; }

// V consecutive channels per thread (V * sizeof(T) = 16 bytes when the channel count allows)
template <typename T, int V> struct Pack { T v[V]; };

template <typename T, int V>
__global__ __launch_bounds__(256) void segment_reduce_kernel(
    const T* __restrict__ src, int c, const int64_t* __restrict__ indices,
    const int64_t* __restrict__ idx_ptr, int64_t m, int op, T* __restrict__ out) {
    const int groups = c / V;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= m * groups) return;
    const int64_t s = e / groups;
    const int ch = (int)(e - s * groups) * V;
    const int64_t b = idx_ptr[s], t = idx_ptr[s + 1];
    float acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = (op == 0) ? -INFINITY : (op == 3 ? INFINITY : 0.f);
    // four members in flight per thread: their row numbers first, then the rows (a member at a time is two
    // dependent latencies each); the reduction keeps the order b, b + 1, ...
    for (int64_t j = b; j < t; j += 4) {
        int64_t row[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) row[u] = indices[j + u < t ? j + u : t - 1];
        Pack<T, V> p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) p[u] = *(const Pack<T, V>*)(src + row[u] * c + ch);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (j + u < t) {
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    const float v = (float)p[u].v[k];
                    acc[k] = (op == 0) ? fmaxf(acc[k], v) : (op == 3 ? fminf(acc[k], v) : acc[k] + v);
                }
            }
        }
    }
    Pack<T, V> r;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float v = acc[k];
        if (op == 1 && t > b) v /= (float)(t - b);
        if (t == b) v = 0.f;
        r.v[k] = (T)v;
    }
    *(Pack<T, V>*)(out + s * c + ch) = r;
}

template <typename T, int V>
__global__ __launch_bounds__(256) void unpool_add_kernel(const T* __restrict__ parent,
                                                         const T* __restrict__ child, int64_t n,
                                                         int c, const int64_t* __restrict__ cluster,
                                                         T* __restrict__ out) {
    const int groups = c / V;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * groups) return;
    const int64_t i = e / groups;
    const int ch = (int)(e - i * groups) * V;
    const Pack<T, V> a = *(const Pack<T, V>*)(parent + i * c + ch);
    const Pack<T, V> b = *(const Pack<T, V>*)(child + cluster[i] * c + ch);
    Pack<T, V> r;
#pragma unroll
    for (int k = 0; k < V; ++k) r.v[k] = (T)((float)a.v[k] + (float)b.v[k]);
    *(Pack<T, V>*)(out + i * c + ch) = r;
}

template <typename T>
void launch_segment_reduce(const void* src, int c, const int64_t* indices, const int64_t* idx_ptr, int64_t m,
                           int op, void* out, hipStream_t stream) {
    constexpr int V = 16 / sizeof(T);
    if (c % V == 0) {
        hipLaunchKernelGGL((segment_reduce_kernel<T, V>), dim3((unsigned)ptv3_ceil_div(m * (c / V), 256)), dim3(256), 0,
                           stream, (const T*)src, c, indices, idx_ptr, m, op, (T*)out);
    } else {
        hipLaunchKernelGGL((segment_reduce_kernel<T, 1>), dim3((unsigned)ptv3_ceil_div(m * c, 256)), dim3(256), 0,
                           stream, (const T*)src, c, indices, idx_ptr, m, op, (T*)out);
    }
}

template <typename T>
void launch_unpool_add(const void* parent, const void* child, int64_t n, int c, const int64_t* cluster, void* out,
                       hipStream_t stream) {
    constexpr int V = 16 / sizeof(T);
    if (c % V == 0) {
        hipLaunchKernelGGL((unpool_add_kernel<T, V>), dim3((unsigned)ptv3_ceil_div(n * (c / V), 256)), dim3(256), 0,
                           stream, (const T*)parent, (const T*)child, n, c, cluster, (T*)out);
    } else {
        hipLaunchKernelGGL((unpool_add_kernel<T, 1>), dim3((unsigned)ptv3_ceil_div(n * c, 256)), dim3(256), 0, stream,
                           (const T*)parent, (const T*)child, n, c, cluster, (T*)out);
    }
}

}  // namespace

extern "C" size_t ptv3_pool_clusters_workspace_bytes(int64_t n) {
    if (n < 0) return 0;
    return ptv3_align256((size_t)(ptv3_ceil_div(n > 0 ? n : 1, PB)) * sizeof(uint32_t));
}

// Per-block cluster counts of ptv3_pool_clusters_static: device memory that belongs to the library's code
// object, one copy per GPU, held until the process ends. 65,536 blocks of 256 points = 256 KiB.
static constexpr int64_t STATIC_MAX_POINTS = (int64_t)1 << 24;
static __device__ __align__(256) uint32_t scratch[STATIC_MAX_POINTS / 256];

namespace {

static_assert(PB == 256, "scratch is sized for 256-point blocks");

int launch_pool_clusters(const int64_t* code0, const int64_t* order0, int64_t n, int shift, const int64_t* offset,
                         int n_scenes, int64_t* cluster, int64_t* idx_ptr, int64_t* head, int64_t* n_clusters,
                         uint32_t* block_cnt, hipStream_t stream) {
    const int64_t blocks = ptv3_ceil_div(n, PB);
    // every one of the `blocks` counts is written by the first kernel before the second reads it: the buffer
    // needs no clearing, whatever an earlier call left in it
    hipLaunchKernelGGL(cluster_count_kernel, dim3((unsigned)blocks), dim3(PB), 0, stream, code0, order0, n,
                       shift, block_cnt);
    hipLaunchKernelGGL(cluster_scan_kernel, dim3(1), dim3(PB), 0, stream, block_cnt, blocks, n_clusters);
    hipLaunchKernelGGL(cluster_assign_kernel, dim3((unsigned)blocks), dim3(PB), 0, stream, code0, order0, n,
                       shift, (const uint32_t*)block_cnt, cluster, idx_ptr, head);
    if (n_scenes > 0)
        hipLaunchKernelGGL(pool_offsets_kernel, dim3((unsigned)ptv3_ceil_div(n_scenes, 256)), dim3(256), 0, stream,
                           offset, n_scenes, order0, (const int64_t*)cluster, n_clusters + 1);
    PTV3_RETURN_LAUNCH();
}

constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
uint32_t* scratch_ptr[MAX_DEVICES];   // device address of `scratch` on each GPU, looked up on first use

// The array's name is a host-side handle, not an address a kernel can use: its address on the current device
// comes from the runtime, once per device.
int static_scratch(uint32_t** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return PTV3_EINVAL;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return PTV3_EINVAL;
        scratch_ptr[dev] = (uint32_t*)p;
    }
    *out = scratch_ptr[dev];
    return PTV3_OK;
}

}  // namespace

extern "C" int ptv3_pool_clusters(const int64_t* code0, const int64_t* order0, int64_t n, int shift,
                                  const int64_t* offset, int n_scenes, int64_t* cluster, int64_t* idx_ptr,
                                  int64_t* head, int64_t* n_clusters, void* workspace, size_t workspace_bytes,
                                  void* stream_) {
    if (n < 1 || n >= (1ll << 31) || shift < 0 || shift > 62 || n_scenes < 0) return PTV3_EINVAL;
    if (n_scenes > 0 && !offset) return PTV3_EINVAL;
    if (!code0 || !order0 || !cluster || !idx_ptr || !head || !n_clusters || !workspace) return PTV3_EINVAL;
    if (workspace_bytes < ptv3_pool_clusters_workspace_bytes(n)) return PTV3_EWORKSPACE;
    return launch_pool_clusters(code0, order0, n, shift, offset, n_scenes, cluster, idx_ptr, head, n_clusters,
                                (uint32_t*)workspace, (hipStream_t)stream_);
}

extern "C" int64_t ptv3_pool_clusters_static_max_points(void) { return STATIC_MAX_POINTS; }

extern "C" int ptv3_pool_clusters_static(const int64_t* code0, const int64_t* order0, int64_t n, int shift,
                                         const int64_t* offset, int n_scenes, int64_t* cluster, int64_t* idx_ptr,
                                         int64_t* head, int64_t* n_clusters, void* stream_) {
    if (n < 0 || shift < 0 || shift > 62 || n_scenes < 0) return PTV3_EINVAL;
    if (n > STATIC_MAX_POINTS) return PTV3_ESTATIC;
    uint32_t* block_cnt = nullptr;
    const int rc = static_scratch(&block_cnt);
    // n == 0: the warm-up call (outside graph capture) that looks the array's address up and launches nothing
    if (rc != PTV3_OK || n == 0) return rc;
    if (n_scenes > 0 && !offset) return PTV3_EINVAL;
    if (!code0 || !order0 || !cluster || !idx_ptr || !head || !n_clusters) return PTV3_EINVAL;
    return launch_pool_clusters(code0, order0, n, shift, offset, n_scenes, cluster, idx_ptr, head, n_clusters,
                                block_cnt, (hipStream_t)stream_);
}

extern "C" int ptv3_pool_gather(const int64_t* code, int64_t n, int k, int shift,
                                const int32_t* grid_coord, int pool_depth, const int64_t* batch,
                                const int64_t* head, int64_t m, const int32_t* row_perm, int64_t* code_out,
                                int32_t* grid_coord_out, int64_t* batch_out, int32_t* indices_out, void* stream) {
    if (n < 0 || m < 0 || m > n || k < 1 || shift < 0 || shift > 62 || pool_depth < 0 || pool_depth > 31)
        return PTV3_EINVAL;
    if (!row_perm_ok(row_perm, k)) return PTV3_EINVAL;
    if (m == 0) return PTV3_OK;
    if (!code || !head || !code_out) return PTV3_EINVAL;
    if ((grid_coord_out && !grid_coord) || (batch_out && !batch) || (indices_out && (!grid_coord || !batch)))
        return PTV3_EINVAL;
    hipLaunchKernelGGL(pool_gather_kernel, dim3((unsigned)ptv3_ceil_div(m, 256)), dim3(256), 0,
                       (hipStream_t)stream, code, n, k, shift, grid_coord, pool_depth, batch, head, m,
                       make_row_perm(row_perm, k), code_out, grid_coord_out, batch_out, indices_out);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_segment_reduce(const void* src, int dtype, int64_t n, int c,
                                   const int64_t* indices, const int64_t* idx_ptr, int64_t m, int op,
                                   void* out, void* stream_) {
    if (n < 0 || m < 0 || c < 1 || op < 0 || op > 3) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (m == 0) return PTV3_OK;
    if (!src || !indices || !idx_ptr || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F32) launch_segment_reduce<float>(src, c, indices, idx_ptr, m, op, out, stream);
    else if (dtype == PTV3_F16) launch_segment_reduce<_Float16>(src, c, indices, idx_ptr, m, op, out, stream);
    else launch_segment_reduce<__bf16>(src, c, indices, idx_ptr, m, op, out, stream);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_unpool_add(const void* parent, const void* child, int dtype, int64_t n, int c,
                               const int64_t* cluster, int64_t m, void* out, void* stream_) {
    if (n < 0 || m < 0 || c < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!parent || !child || !cluster || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F32) launch_unpool_add<float>(parent, child, n, c, cluster, out, stream);
    else if (dtype == PTV3_F16) launch_unpool_add<_Float16>(parent, child, n, c, cluster, out, stream);
    else launch_unpool_add<__bf16>(parent, child, n, c, cluster, out, stream);
    PTV3_RETURN_LAUNCH();
}

extern "C" size_t ptv3_pool_orders_workspace_bytes(int64_t n, int k) {
    if (n < 0 || k < 1) return 0;
    return ptv3_align256((size_t)k * ptv3_ceil_div(n > 0 ? n : 1, PB) * sizeof(uint32_t));
}

extern "C" int ptv3_pool_orders(const int64_t* order, const int64_t* cluster, int64_t n, int k, int64_t m,
                                const int32_t* row_perm, int64_t* order_out, int64_t* inverse_out, void* workspace,
                                size_t workspace_bytes, void* stream_) {
    if (n < 1 || n >= (1ll << 31) || k < 1 || k > 65535 || m < 1 || m > n) return PTV3_EINVAL;
    if (!row_perm_ok(row_perm, k)) return PTV3_EINVAL;
    const RowPerm perm = make_row_perm(row_perm, k);
    if (!order || !cluster || !order_out || !inverse_out || !workspace) return PTV3_EINVAL;
    if (workspace_bytes < ptv3_pool_orders_workspace_bytes(n, k)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const int64_t blocks = ptv3_ceil_div(n, PB);
    uint32_t* block_cnt = (uint32_t*)workspace;
    const dim3 grid((unsigned)blocks, (unsigned)k);
    hipLaunchKernelGGL(order_count_kernel, grid, dim3(PB), 0, stream, order, cluster, n, perm, block_cnt);
    hipLaunchKernelGGL(order_scan_kernel, dim3((unsigned)k), dim3(PB), 0, stream, block_cnt, blocks);
    hipLaunchKernelGGL(order_assign_kernel, grid, dim3(PB), 0, stream, order, cluster, n, m, perm,
                       (const uint32_t*)block_cnt, order_out, inverse_out);
    PTV3_RETURN_LAUNCH();
}
