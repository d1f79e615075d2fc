// Voxel hash shared by the neighbour-map and the pair-list builders.
//
// What bounds a neighbour search on the GPU is the number of distinct cache lines requested, not
// bytes: a 5x5x5 search that probes a per-voxel hash 125 times per voxel runs at the L2's request
// rate. The table here is therefore keyed on 4x4x4 BLOCKS of voxels: a 16-byte header {block key,
// 64-bit occupancy mask} found by open addressing (linear probing, load <= 2/3), and 64 row
// indices per block that are only valid where the mask has a bit. The 3^3 (5^3) neighbourhood of
// a voxel touches at most 8 blocks, so a voxel reads at most 8 headers, learns from the masks
// exactly which neighbours exist (no false positives, no per-neighbour probe), and reads one row
// index per existing neighbour: ~13 requests per voxel for 5^3 on a surface scan instead of 125.
#pragma once
#include "common.h"

namespace {

constexpr uint64_t VH_EMPTY = ~0ull;
constexpr int VH_SHIFT = 4;   // coordinates are shifted by this before blocking, so x - 2 stays >= 0

struct __align__(16) VoxelBlock {
    uint64_t key;    // (batch, xs >> 2, ys >> 2, zs >> 2)
    uint64_t mask;   // bit (xs & 3) << 4 | (ys & 3) << 2 | (zs & 3)
};

struct VoxelHash {
    VoxelBlock* blocks;   // cap headers
    int32_t* rows;        // cap * 64 row indices
    uint32_t mask;        // cap - 1
};

__device__ __forceinline__ uint64_t vh_block_key(int b, int bx, int by, int bz) {
    return ((uint64_t)(uint32_t)b << 48) | ((uint64_t)(uint32_t)bx << 32) | ((uint64_t)(uint32_t)by << 16) |
           (uint64_t)(uint32_t)bz;
}

__device__ __forceinline__ uint64_t vh_mix(uint64_t k) {
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdull;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ull;
    k ^= k >> 33;
    return k;
}

__device__ __forceinline__ VoxelBlock vh_load(const VoxelHash& h, uint32_t slot) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 w = *(const u32x4*)&h.blocks[slot];
    VoxelBlock s;
    s.key = (uint64_t)w[0] | ((uint64_t)w[1] << 32);
    s.mask = (uint64_t)w[2] | ((uint64_t)w[3] << 32);
    return s;
}

// bits of a block mask whose local coordinate along one axis lies in [lo, hi] (clamped to 0..3);
// `unit` is the bit stride of the axis inside the mask (16, 4, 1) and `rep` repeats the pattern
// over the other axes
__device__ __forceinline__ uint64_t vh_axis_bits(int lo, int hi, int unit, uint64_t rep) {
    lo = lo < 0 ? 0 : lo;
    hi = hi > 3 ? 3 : hi;
    if (hi < lo) return 0;
    const int width = unit * (hi - lo + 1);   // <= 64
    const uint64_t span = (width >= 64 ? ~0ull : ((1ull << width) - 1ull)) << (unit * lo);
    return span * rep;
}

// The up-to-8 blocks around a voxel, their header slots and the occupied cells of each that lie
// inside the voxel's (2r+1)^3 window.
struct VoxelWindow {
    uint32_t slot[8];
    uint64_t hits[8];
    int bx0, by0, bz0;   // block coordinates of block 0
};

template <int R>
__device__ __forceinline__ VoxelWindow vh_window(const VoxelHash& h, int b, int x, int y, int z) {
    const int xs = x + VH_SHIFT, ys = y + VH_SHIFT, zs = z + VH_SHIFT;
    VoxelWindow w;
    w.bx0 = (xs - R) >> 2;
    w.by0 = (ys - R) >> 2;
    w.bz0 = (zs - R) >> 2;
    const int nx = ((xs + R) >> 2) - w.bx0, ny = ((ys + R) >> 2) - w.by0, nz = ((zs + R) >> 2) - w.bz0;   // 0 or 1
    uint64_t key[8];
    VoxelBlock cur[8];
    bool live[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int ox = k >> 2, oy = (k >> 1) & 1, oz = k & 1;
        live[k] = ox <= nx && oy <= ny && oz <= nz;
        key[k] = vh_block_key(b, w.bx0 + ox, w.by0 + oy, w.bz0 + oz);
        w.slot[k] = (uint32_t)vh_mix(key[k]) & h.mask;
        w.hits[k] = 0;
        cur[k].key = VH_EMPTY;
        cur[k].mask = 0;
        if (live[k]) cur[k] = vh_load(h, w.slot[k]);   // all first probes in flight together
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if (!live[k]) continue;
        const int ox = k >> 2, oy = (k >> 1) & 1, oz = k & 1;
        uint64_t m = 0;
        for (uint32_t probe = 0; probe <= h.mask; ++probe) {
            if (cur[k].key == key[k]) { m = cur[k].mask; break; }
            if (cur[k].key == VH_EMPTY) break;
            w.slot[k] = (w.slot[k] + 1) & h.mask;
            cur[k] = vh_load(h, w.slot[k]);
        }
        // window in this block's local coordinates
        const int lx = xs - R - 4 * (w.bx0 + ox), ly = ys - R - 4 * (w.by0 + oy), lz = zs - R - 4 * (w.bz0 + oz);
        w.hits[k] = m & vh_axis_bits(lx, lx + 2 * R, 16, 1ull) & vh_axis_bits(ly, ly + 2 * R, 4, 0x0001000100010001ull) &
                    vh_axis_bits(lz, lz + 2 * R, 1, 0x1111111111111111ull);
    }
    return w;
}

// tap index (kx * ks + ky) * ks + kz of cell `bit` of block k of the window of a voxel at (x, y, z)
template <int R>
__device__ __forceinline__ int vh_tap_of(const VoxelWindow& w, int k, int bit, int x, int y, int z) {
    constexpr int KS = 2 * R + 1;
    const int cx = 4 * (w.bx0 + (k >> 2)) + (bit >> 4) - VH_SHIFT;
    const int cy = 4 * (w.by0 + ((k >> 1) & 1)) + ((bit >> 2) & 3) - VH_SHIFT;
    const int cz = 4 * (w.bz0 + (k & 1)) + (bit & 3) - VH_SHIFT;
    return ((cx - x + R) * KS + (cy - y + R)) * KS + (cz - z + R);
}

__global__ __launch_bounds__(256) void vh_fill_kernel(VoxelHash h, int64_t cap) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < cap) {
        h.blocks[i].key = VH_EMPTY;
        h.blocks[i].mask = 0;
    }
}

__global__ __launch_bounds__(256) void vh_insert_kernel(const int32_t* __restrict__ indices, int64_t n, VoxelHash h) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int4 v = ((const int4*)indices)[i];
    const int xs = v.y + VH_SHIFT, ys = v.z + VH_SHIFT, zs = v.w + VH_SHIFT;
    const uint64_t key = vh_block_key(v.x, xs >> 2, ys >> 2, zs >> 2);
    const int bit = (xs & 3) << 4 | (ys & 3) << 2 | (zs & 3);
    uint32_t slot = (uint32_t)vh_mix(key) & h.mask;
    for (uint32_t probe = 0; probe <= h.mask; ++probe) {
        const uint64_t prev = atomicCAS((unsigned long long*)&h.blocks[slot].key, (unsigned long long)VH_EMPTY,
                                        (unsigned long long)key);
        if (prev == VH_EMPTY || prev == key) {
            atomicOr((unsigned long long*)&h.blocks[slot].mask, 1ull << bit);
            h.rows[(int64_t)slot * 64 + bit] = (int32_t)i;
            return;
        }
        slot = (slot + 1) & h.mask;
    }
}

// headers for the worst case of one voxel per block at load <= 2/3
inline int64_t vh_capacity(int64_t n) {
    int64_t cap = 1024;
    while (2 * cap < 3 * n) cap <<= 1;
    return cap;
}

inline size_t vh_bytes(int64_t n) {
    const int64_t cap = vh_capacity(n);
    return ptv3_align256((size_t)cap * sizeof(VoxelBlock)) + ptv3_align256((size_t)cap * 64 * sizeof(int32_t));
}

// the table carved out of `base` (vh_bytes(n) bytes)
inline VoxelHash vh_view(void* base, int64_t n) {
    const int64_t cap = vh_capacity(n);
    VoxelHash h;
    h.blocks = (VoxelBlock*)base;
    h.rows = (int32_t*)((char*)base + ptv3_align256((size_t)cap * sizeof(VoxelBlock)));
    h.mask = (uint32_t)(cap - 1);
    return h;
}

// carve and launch fill + insert (the row indices need no initialisation: the masks say which are valid)
inline VoxelHash vh_build(void* base, const int32_t* indices, int64_t n, hipStream_t stream) {
    const VoxelHash h = vh_view(base, n);
    const int64_t cap = vh_capacity(n);
    hipLaunchKernelGGL(vh_fill_kernel, dim3((unsigned)ptv3_ceil_div(cap, 256)), dim3(256), 0, stream, h, cap);
    hipLaunchKernelGGL(vh_insert_kernel, dim3((unsigned)ptv3_ceil_div(n, 256)), dim3(256), 0, stream, indices, n, h);
    return h;
}

}  // namespace
