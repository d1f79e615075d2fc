// Voxelisation in front of the model: coordinates -> grid coordinates, one point kept per voxel.
//
// What Pointcept's data pipeline does on the host before PointTransformerV3.forward sees a batch
// (the model's own fallback, model.py:88-96, only derives grid_coord): per scene,
// grid_coord = floor((coord - min over the scene) / grid_size), and of the points that fall into one
// voxel the first in input order is kept. Here on the device, in input order, deterministic:
//   scene_min   per-scene minimum of every axis (wave reduction, one atomic per wave and axis);
//   insert      open-addressing table keyed (scene, x, y, z); atomicMin leaves the first point of
//               every voxel in its slot;
//   count/scan/assign   kept flags -> positions (three-kernel scan), the kept points' grid
//               coordinates and indices, the scene ends of the kept points;
//   inverse     voxel of every input point.
#include "voxelhash.h"

namespace {

constexpr int VX_THREADS = 256;
constexpr int VX_WAVES = VX_THREADS / PTV3_WAVE;
constexpr uint64_t VX_EMPTY = ~0ull;

struct VoxWs {
    uint64_t* keys;       // [cap]
    int32_t* first;       // [cap] lowest rank among the voxel's points (seed 0: lowest point index)
    int32_t* voxel;       // [cap] position of the voxel among the kept points
    int32_t* slot_of;     // [n]
    uint32_t* block_cnt;  // [blocks]
    uint32_t* scene_min;  // [nb][3] order-preserving encoding of the float minimum
    int32_t* status;      // [1] non-zero: a grid coordinate does not fit 16 bits
    int64_t cap;
    size_t bytes;
};

int64_t vx_capacity(int64_t n) {
    int64_t cap = 1024;
    while (cap < 2 * n) cap <<= 1;
    return cap;
}

VoxWs vx_carve(void* base, int64_t n, int nb) {
    VoxWs w;
    char* p = (char*)base;
    size_t off = 0;
    w.cap = vx_capacity(n);
    const int64_t blocks = ptv3_ceil_div(n > 0 ? n : 1, VX_THREADS);
    w.keys = (uint64_t*)(p + off); off += ptv3_align256((size_t)w.cap * 8);
    w.first = (int32_t*)(p + off); off += ptv3_align256((size_t)w.cap * 4);
    w.voxel = (int32_t*)(p + off); off += ptv3_align256((size_t)w.cap * 4);
    w.slot_of = (int32_t*)(p + off); off += ptv3_align256((size_t)(n > 0 ? n : 1) * 4);
    w.block_cnt = (uint32_t*)(p + off); off += ptv3_align256((size_t)blocks * 4);
    w.scene_min = (uint32_t*)(p + off); off += ptv3_align256((size_t)(nb > 0 ? nb : 1) * 3 * 4);
    w.status = (int32_t*)(p + off); off += 256;
    w.bytes = off;
    return w;
}

// floats order like these unsigned integers
__device__ __forceinline__ uint32_t f2ord(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ord2f(uint32_t u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// scene of point i: the first scene whose end is > i
__device__ __forceinline__ int scene_of(const int64_t* __restrict__ offset, int nb, int64_t i) {
    int lo = 0, hi = nb;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (offset[mid] <= i) lo = mid + 1; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(VX_THREADS) void vx_init_kernel(VoxWs w, int nb, int64_t* __restrict__ offset_out) {
    const int64_t i = (int64_t)blockIdx.x * VX_THREADS + threadIdx.x;
    if (i < w.cap) {
        w.keys[i] = VX_EMPTY;
        w.first[i] = 0x7fffffff;
    }
    if (i < 3 * (int64_t)nb) w.scene_min[i] = 0xffffffffu;
    if (i < nb) offset_out[i] = 0;
    if (i == 0) w.status[0] = 0;
}

constexpr int VX_MIN_ITERS = 16;   // points per thread of the minimum kernel

// A wave walks VX_MIN_ITERS * 64 consecutive points and almost always stays inside one scene: lanes
// keep running minima and the wave issues three atomics when the scene changes and at the end
// (a few thousand atomics per call; one per wave and point block serialised on a dozen addresses).
__global__ __launch_bounds__(VX_THREADS) void vx_scene_min_kernel(const float* __restrict__ coord, int64_t n,
                                                                  const int64_t* __restrict__ offset, int nb, VoxWs w) {
    const int lane = threadIdx.x % PTV3_WAVE;
    const int64_t wave_id = (int64_t)blockIdx.x * VX_WAVES + threadIdx.x / PTV3_WAVE;
    const int64_t base = wave_id * (VX_MIN_ITERS * PTV3_WAVE);
    int cur = -1;   // scene of the running minima (uniform over the wave)
    uint32_t m[3] = {0xffffffffu, 0xffffffffu, 0xffffffffu};
    auto flush = [&]() {
        if (cur < 0) return;
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            uint32_t r = m[a];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) r = min(r, (uint32_t)__shfl_xor((int)r, off, PTV3_WAVE));
            if (lane == 0) atomicMin(&w.scene_min[3 * cur + a], r);
            m[a] = 0xffffffffu;
        }
    };
    for (int it = 0; it < VX_MIN_ITERS; ++it) {
        const int64_t i = base + (int64_t)it * PTV3_WAVE + lane;
        if (base + (int64_t)it * PTV3_WAVE >= n) break;   // uniform
        const bool live = i < n;
        const int s = live ? scene_of(offset, nb, i) : -1;
        uint32_t v[3] = {0xffffffffu, 0xffffffffu, 0xffffffffu};
        if (live) {
#pragma unroll
            for (int a = 0; a < 3; ++a) v[a] = f2ord(coord[3 * i + a]);
        }
        const int s0 = __shfl(s, 0, PTV3_WAVE);   // lane 0 is live whenever the iteration runs
        const bool uniform = __ballot(live && s != s0) == 0;
        if (uniform && s0 == cur) {
#pragma unroll
            for (int a = 0; a < 3; ++a) m[a] = min(m[a], v[a]);
            continue;
        }
        flush();
        if (uniform) {
            cur = s0;
#pragma unroll
            for (int a = 0; a < 3; ++a) m[a] = v[a];
        } else {
            cur = -1;
            if (live) {
#pragma unroll
                for (int a = 0; a < 3; ++a) atomicMin(&w.scene_min[3 * s + a], v[a]);
            }
        }
    }
    flush();
}

__device__ __forceinline__ void vx_grid(const float* __restrict__ coord, int64_t i, int s, const VoxWs& w, float grid_size,
                                        int32_t (&g)[3]) {
#pragma unroll
    for (int a = 0; a < 3; ++a) g[a] = (int32_t)floorf((coord[3 * i + a] - ord2f(w.scene_min[3 * s + a])) / grid_size);
}

// Rank of point i among the points of its voxel: the point with the lowest rank is kept. Seed 0: the
// index itself (the first point in input order, GridSample's test mode). Otherwise a bijection of the
// 32-bit index keyed by the seed (odd multiplications and xor-shifts, each invertible), so ranks never tie
// and the lowest belongs to a member drawn uniformly -- GridSample's train mode, which takes a random
// member of every voxel.
__device__ __forceinline__ int32_t vx_rank(int64_t i, uint32_t seed) {
    uint32_t x = (uint32_t)i;
    if (seed != 0u) {
        x ^= seed;
        x *= 0x9E3779B1u;
        x ^= x >> 15;
        x *= 0x85EBCA77u;
        x ^= x >> 13;
        x *= 0xC2B2AE3Du;
        x ^= x >> 16;
        x += seed * 0x27D4EB2Fu;
    }
    return (int32_t)x;
}

__global__ __launch_bounds__(VX_THREADS) void vx_insert_kernel(const float* __restrict__ coord, int64_t n,
                                                               const int64_t* __restrict__ offset, int nb,
                                                               float grid_size, VoxWs w, uint32_t seed) {
    const int64_t i = (int64_t)blockIdx.x * VX_THREADS + threadIdx.x;
    if (i >= n) return;
    const int s = scene_of(offset, nb, i);
    int32_t g[3];
    vx_grid(coord, i, s, w, grid_size, g);
    if ((g[0] | g[1] | g[2]) >> 16) w.status[0] = 1;   // (negative cannot happen: the minimum is subtracted)
    const uint64_t key = vh_block_key(s, g[0], g[1], g[2]);
    const uint32_t mask = (uint32_t)(w.cap - 1);
    uint32_t slot = (uint32_t)vh_mix(key) & mask;
    for (uint32_t probe = 0; probe <= mask; ++probe) {
        const uint64_t prev = atomicCAS((unsigned long long*)&w.keys[slot], (unsigned long long)VX_EMPTY,
                                        (unsigned long long)key);
        if (prev == VX_EMPTY || prev == key) {
            atomicMin(&w.first[slot], vx_rank(i, seed));
            w.slot_of[i] = (int32_t)slot;
            return;
        }
        slot = (slot + 1) & mask;
    }
}

__device__ __forceinline__ uint32_t vx_block_scan(uint32_t v, uint32_t* total) {
    __shared__ uint32_t wsum[VX_WAVES];
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
    for (int k = 0; k < VX_WAVES; ++k) {
        const uint32_t c = wsum[k];
        if (k < wave) base += c;
        tot += c;
    }
    *total = tot;
    __syncthreads();
    return x + base;
}

__global__ __launch_bounds__(VX_THREADS) void vx_count_kernel(int64_t n, VoxWs w, uint32_t seed) {
    const int64_t i = (int64_t)blockIdx.x * VX_THREADS + threadIdx.x;
    const uint32_t keep = (i < n && w.first[w.slot_of[i]] == vx_rank(i, seed)) ? 1u : 0u;
    uint32_t total;
    vx_block_scan(keep, &total);
    if (threadIdx.x == 0) w.block_cnt[blockIdx.x] = total;
}

// one block: exclusive scan of the block counts in place, total (+ status) to counts[0], counts[1]
__global__ __launch_bounds__(VX_THREADS) void vx_scan_kernel(VoxWs w, int64_t blocks, int64_t* __restrict__ counts) {
    uint32_t carry = 0;
    for (int64_t b0 = 0; b0 < blocks; b0 += VX_THREADS) {
        const int64_t b = b0 + threadIdx.x;
        const uint32_t v = b < blocks ? w.block_cnt[b] : 0u;
        uint32_t total;
        const uint32_t inc = vx_block_scan(v, &total);
        if (b < blocks) w.block_cnt[b] = carry + inc - v;
        carry += total;
    }
    if (threadIdx.x == 0) {
        counts[0] = (int64_t)carry;
        counts[1] = (int64_t)w.status[0];
    }
}

__global__ __launch_bounds__(VX_THREADS) void vx_assign_kernel(const float* __restrict__ coord, int64_t n,
                                                               const int64_t* __restrict__ offset, int nb,
                                                               float grid_size, VoxWs w, int32_t* __restrict__ grid_out,
                                                               int64_t* __restrict__ index_out,
                                                               int64_t* __restrict__ offset_out, uint32_t seed) {
    const int64_t i = (int64_t)blockIdx.x * VX_THREADS + threadIdx.x;
    const bool live = i < n;
    const int32_t slot = live ? w.slot_of[i] : 0;
    const bool keep = live && w.first[slot] == vx_rank(i, seed);
    uint32_t total;
    const uint32_t inc = vx_block_scan(keep ? 1u : 0u, &total);
    if (!live) return;
    const int64_t upto = (int64_t)w.block_cnt[blockIdx.x] + inc;   // kept points among 0..i
    if (keep) {
        const int64_t pos = upto - 1;
        const int s = scene_of(offset, nb, i);
        int32_t g[3];
        vx_grid(coord, i, s, w, grid_size, g);
#pragma unroll
        for (int a = 0; a < 3; ++a) grid_out[3 * pos + a] = g[a];
        index_out[pos] = i;
        w.voxel[slot] = (int32_t)pos;
    }
    // the scenes that end with point i (several when empty scenes follow) end with `upto` kept points
    int b = scene_of(offset, nb, i);   // offset[b] > i
    while (b < nb && offset[b] == i + 1) offset_out[b++] = upto;
}

__global__ __launch_bounds__(VX_THREADS) void vx_inverse_kernel(int64_t n, VoxWs w, int64_t* __restrict__ inverse) {
    const int64_t i = (int64_t)blockIdx.x * VX_THREADS + threadIdx.x;
    if (i < n) inverse[i] = w.voxel[w.slot_of[i]];
}

}  // namespace

extern "C" size_t ptv3_voxelize_workspace_bytes(int64_t n, int n_scenes) {
    if (n < 0 || n_scenes < 1) return 0;
    return vx_carve(nullptr, n, n_scenes).bytes;
}

extern "C" int ptv3_voxelize(const float* coord, int64_t n, const int64_t* offset, int n_scenes, float grid_size,
                             int32_t* grid_coord, int64_t* index, int64_t* inverse, int64_t* offset_out,
                             int64_t* counts, uint32_t pick_seed, void* workspace, size_t workspace_bytes,
                             void* stream_) {
    if (n < 1 || n >= (1ll << 30) || n_scenes < 1 || n_scenes > 65535 || !(grid_size > 0.f)) return PTV3_EINVAL;
    if (!coord || !offset || !grid_coord || !index || !offset_out || !counts || !workspace) return PTV3_EINVAL;
    VoxWs w = vx_carve(workspace, n, n_scenes);
    if (workspace_bytes < w.bytes) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const int64_t blocks = ptv3_ceil_div(n, VX_THREADS);
    const int64_t init = w.cap > 3 * (int64_t)n_scenes ? w.cap : 3 * (int64_t)n_scenes;
    hipLaunchKernelGGL(vx_init_kernel, dim3((unsigned)ptv3_ceil_div(init, VX_THREADS)), dim3(VX_THREADS), 0, stream, w,
                       n_scenes, offset_out);
    hipLaunchKernelGGL(vx_scene_min_kernel, dim3((unsigned)ptv3_ceil_div(n, VX_THREADS * VX_MIN_ITERS)), dim3(VX_THREADS),
                       0, stream, coord, n, offset, n_scenes, w);
    hipLaunchKernelGGL(vx_insert_kernel, dim3((unsigned)blocks), dim3(VX_THREADS), 0, stream, coord, n, offset,
                       n_scenes, grid_size, w, pick_seed);
    hipLaunchKernelGGL(vx_count_kernel, dim3((unsigned)blocks), dim3(VX_THREADS), 0, stream, n, w, pick_seed);
    hipLaunchKernelGGL(vx_scan_kernel, dim3(1), dim3(VX_THREADS), 0, stream, w, blocks, counts);
    hipLaunchKernelGGL(vx_assign_kernel, dim3((unsigned)blocks), dim3(VX_THREADS), 0, stream, coord, n, offset,
                       n_scenes, grid_size, w, grid_coord, index, offset_out, pick_seed);
    if (inverse)
        hipLaunchKernelGGL(vx_inverse_kernel, dim3((unsigned)blocks), dim3(VX_THREADS), 0, stream, n, w, inverse);
    PTV3_RETURN_LAUNCH();
}
