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
//
// The pair lists can also be built straight from the voxel coordinates (ptv3_kmap_plan_*): the same
// two scans, with the activity mask looked up in the voxel hash on the fly instead of read from a
// stored map. For a 5x5x5 stem on 400k voxels the stored map is 200 MB written once and read twice
// for ~6 active taps of 125 per voxel; the direct form never materialises it.
#include "voxelhash.h"

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
// A column is one sequential chain of block scans, so the work-group is as wide as it gets
// (1024 threads: a 400k-voxel level is 7 steps instead of 25).
constexpr int SCAN_THREADS = 1024;
constexpr int SCAN_WAVES = SCAN_THREADS / PTV3_WAVE;

__global__ __launch_bounds__(SCAN_THREADS) void plan_scan_kernel(uint32_t* __restrict__ blk_tap_cnt,
                                                                 uint32_t* __restrict__ blk_row_sum,
                                                                 int64_t blocks, int taps,
                                                                 uint32_t* __restrict__ tap_total,
                                                                 int64_t* __restrict__ n_pairs) {
    __shared__ uint32_t wsum[SCAN_WAVES];
    const int col = blockIdx.x;
    const int lane = threadIdx.x % PTV3_WAVE, wave = threadIdx.x / PTV3_WAVE;
    uint32_t carry = 0;
    for (int64_t b0 = 0; b0 < blocks; b0 += SCAN_THREADS) {
        const int64_t b = b0 + threadIdx.x;
        uint32_t* p = col < taps ? &blk_tap_cnt[b * taps + col] : &blk_row_sum[b];
        const uint32_t v = b < blocks ? *p : 0u;
        uint32_t x = v;
#pragma unroll
        for (int off = 1; off < PTV3_WAVE; off <<= 1) {
            const uint32_t y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        if (lane == PTV3_WAVE - 1) wsum[wave] = x;
        __syncthreads();
        // the 16 wave totals: every wave scans them itself (lanes 0..15)
        uint32_t ws = lane < SCAN_WAVES ? wsum[lane] : 0u;
#pragma unroll
        for (int off = 1; off < SCAN_WAVES; off <<= 1) {
            const uint32_t y = __shfl_up(ws, off, PTV3_WAVE);
            if (lane >= off) ws += y;
        }
        const uint32_t total = __shfl(ws, SCAN_WAVES - 1, PTV3_WAVE);
        const uint32_t base = wave == 0 ? 0u : __shfl(ws, wave - 1, PTV3_WAVE);
        if (b < blocks) *p = carry + base + x - v;
        carry += total;
        __syncthreads();
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

PlanWs carve_plan(void* base, int64_t n, int taps, int block_threads = PLAN_THREADS) {
    const int64_t blocks = ptv3_ceil_div(n > 0 ? n : 1, block_threads);
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


// ---- pair lists straight from the voxel hash: one wave per block of 64 voxels, thread = voxel.
// A lane reads the headers of the (at most 8) voxel blocks around its voxel, all in flight
// together, and knows from their masks which taps exist. Found taps are published as per-tap lane
// masks in LDS, which give the block's per-tap counts (count pass) and every pair's rank inside
// (block, tap) (fill pass); the fill pass then reads one row index per existing neighbour.
constexpr int DIRECT_THREADS = PTV3_WAVE;

struct TapSet {
    uint64_t lo, hi;   // bit t <-> tap t (< 128)
    __device__ __forceinline__ void set(int t) {
        if (t < 64) lo |= 1ull << t; else hi |= 1ull << (t - 64);
    }
    __device__ __forceinline__ int count() const { return __popcll(lo) + __popcll(hi); }
    __device__ __forceinline__ int rank(int t) const {   // members below t
        return t < 64 ? __popcll(lo & ((1ull << t) - 1ull)) : __popcll(lo) + __popcll(hi & ((1ull << (t - 64)) - 1ull));
    }
};

__device__ __forceinline__ uint32_t wave_scan_incl(uint32_t v, uint32_t* total) {
    const int lane = threadIdx.x % PTV3_WAVE;
    uint32_t x = v;
#pragma unroll
    for (int off = 1; off < PTV3_WAVE; off <<= 1) {
        const uint32_t y = __shfl_up(x, off, PTV3_WAVE);
        if (lane >= off) x += y;
    }
    *total = __shfl(x, PTV3_WAVE - 1, PTV3_WAVE);
    return x;
}

// taps of the window that exist, also published in lane_mask[t]
template <int KS>
__device__ __forceinline__ TapSet publish_taps(const VoxelWindow& w, int4 v, unsigned long long* lane_mask) {
    const int lane = threadIdx.x;
    TapSet found = {0, 0};
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        uint64_t m = w.hits[k];
        while (m) {
            const int bit = __builtin_ctzll(m);
            m &= m - 1;
            const int t = vh_tap_of<KS / 2>(w, k, bit, v.y, v.z, v.w);
            found.set(t);
            atomicOr(&lane_mask[t], 1ull << lane);
        }
    }
    return found;
}

// what the count pass leaves per voxel for the fill pass: the header slots of its 8 blocks and
// its found taps, as arrays over the voxels (coalesced both ways)
struct DirectNotes {
    uint32_t* slot;     // [8][n]
    uint64_t* found;    // [2][n]
};

template <int KS>
__global__ __launch_bounds__(DIRECT_THREADS) void direct_count_kernel(
    const int32_t* __restrict__ indices, int64_t n, VoxelHash h, DirectNotes notes, uint32_t* __restrict__ row_cnt,
    uint32_t* __restrict__ blk_row_sum, uint32_t* __restrict__ blk_tap_cnt) {
    constexpr int TAPS = KS * KS * KS;
    __shared__ unsigned long long lane_mask[MAX_TAPS];
    const int lane = threadIdx.x;
    const int64_t i = (int64_t)blockIdx.x * DIRECT_THREADS + lane;
    lane_mask[lane] = 0;
    lane_mask[lane + 64] = 0;
    __syncthreads();
    uint32_t cnt = 0;
    if (i < n) {
        const int4 v = ((const int4*)indices)[i];
        const VoxelWindow w = vh_window<KS / 2>(h, v.x, v.y, v.z, v.w);
        const TapSet found = publish_taps<KS>(w, v, lane_mask);
        cnt = (uint32_t)found.count();
        row_cnt[i] = cnt;
#pragma unroll
        for (int k = 0; k < 8; ++k) notes.slot[(int64_t)k * n + i] = w.slot[k];
        notes.found[i] = found.lo;
        notes.found[n + i] = found.hi;
    }
    uint32_t total;
    wave_scan_incl(cnt, &total);
    if (lane == 0) blk_row_sum[blockIdx.x] = total;
    __syncthreads();
    for (int t = lane; t < TAPS; t += DIRECT_THREADS)
        blk_tap_cnt[(int64_t)blockIdx.x * TAPS + t] = (uint32_t)__popcll(lane_mask[t]);
}

constexpr int DIRECT_STAGE = 1024;   // pairs of one 64-voxel block staged in LDS for coalesced writes

template <int KS>
__global__ __launch_bounds__(DIRECT_THREADS) void direct_fill_kernel(
    const int32_t* __restrict__ indices, int64_t n, VoxelHash h, DirectNotes notes, const uint32_t* __restrict__ row_cnt,
    const uint32_t* __restrict__ blk_row_off, const uint32_t* __restrict__ blk_tap_off,
    const int32_t* __restrict__ tap_ptr, int32_t* __restrict__ row_ptr, int32_t* __restrict__ pair_in,
    int32_t* __restrict__ pair_slot) {
    constexpr int R = KS / 2, TAPS = KS * KS * KS, CENTRE = TAPS / 2;
    __shared__ unsigned long long lane_mask[MAX_TAPS];
    __shared__ uint32_t tap_base[MAX_TAPS];    // first pair of (block, tap) in the tap-major lists
    __shared__ uint32_t tap_start[MAX_TAPS];   // first pair of (block, tap) in the staging buffer
    __shared__ uint32_t blk_slot[8][DIRECT_THREADS];
    __shared__ uint32_t stage_q[DIRECT_STAGE];
    __shared__ int32_t stage_in[DIRECT_STAGE], stage_slot[DIRECT_STAGE];
    const int lane = threadIdx.x;
    const int64_t i = (int64_t)blockIdx.x * DIRECT_THREADS + lane;
    const uint64_t below = (1ull << lane) - 1ull;
    lane_mask[lane] = 0;
    lane_mask[lane + 64] = 0;
    for (int t = lane; t < TAPS; t += DIRECT_THREADS)
        tap_base[t] = (uint32_t)tap_ptr[t] + blk_tap_off[(int64_t)blockIdx.x * TAPS + t];
    const uint32_t cnt = i < n ? row_cnt[i] : 0u;
    uint32_t total;
    const uint32_t inc = wave_scan_incl(cnt, &total);
    const uint32_t slot0 = blk_row_off[blockIdx.x] + inc - cnt;   // first output slot of my voxel
    if (i < n) row_ptr[i] = (int32_t)slot0;
    if (i == n - 1) row_ptr[n] = (int32_t)(slot0 + cnt);
    int4 v = {0, 0, 0, 0};
    TapSet found = {0, 0};
    if (i < n) {
        v = ((const int4*)indices)[i];
        found.lo = notes.found[i];
        found.hi = notes.found[n + i];
#pragma unroll
        for (int k = 0; k < 8; ++k) blk_slot[k][lane] = notes.slot[(int64_t)k * n + i];
    }
    __syncthreads();
    // per-tap lane masks from the found sets
    {
        TapSet f = found;
        while (f.lo) { const int t = __builtin_ctzll(f.lo); f.lo &= f.lo - 1; atomicOr(&lane_mask[t], 1ull << lane); }
        while (f.hi) { const int t = 64 + __builtin_ctzll(f.hi); f.hi &= f.hi - 1; atomicOr(&lane_mask[t], 1ull << lane); }
    }
    __syncthreads();
    // staging position of every tap's first pair: exclusive scan of the per-tap counts
    {
        const uint32_t c0 = (uint32_t)__popcll(lane_mask[lane]), c1 = (uint32_t)__popcll(lane_mask[lane + 64]);
        uint32_t t0, t1;
        const uint32_t i0 = wave_scan_incl(c0, &t0);
        const uint32_t i1 = wave_scan_incl(c1, &t1);
        tap_start[lane] = i0 - c0;
        tap_start[lane + 64] = t0 + i1 - c1;
    }
    __syncthreads();
    const bool staged = total <= (uint32_t)DIRECT_STAGE;   // total = pairs of this block
    // a voxel's slots follow tap order, a tap's pairs voxel order: both ranks come from the masks
    const int xs = v.y + VH_SHIFT, ys = v.z + VH_SHIFT, zs = v.w + VH_SHIFT;
    const int bx0 = (xs - R) >> 2, by0 = (ys - R) >> 2, bz0 = (zs - R) >> 2;
    TapSet f = found;
    uint32_t slot = slot0;
    while (f.lo | f.hi) {
        int t;
        if (f.lo) { t = __builtin_ctzll(f.lo); f.lo &= f.lo - 1; }
        else { t = 64 + __builtin_ctzll(f.hi); f.hi &= f.hi - 1; }
        int32_t src = (int32_t)i;
        if (t != CENTRE) {
            const int cx = xs + t / (KS * KS) - R, cy = ys + (t / KS) % KS - R, cz = zs + t % KS - R;
            const int k = ((cx >> 2) - bx0) << 2 | ((cy >> 2) - by0) << 1 | ((cz >> 2) - bz0);
            const int bit = (cx & 3) << 4 | (cy & 3) << 2 | (cz & 3);
            src = h.rows[(int64_t)blk_slot[k][lane] * 64 + bit];
        }
        const uint32_t rank = (uint32_t)__popcll(lane_mask[t] & below);
        const uint32_t q = tap_base[t] + rank;
        if (staged) {
            const uint32_t e = tap_start[t] + rank;
            stage_q[e] = q;
            stage_in[e] = src;
            stage_slot[e] = (int32_t)slot;
        } else {
            pair_in[q] = src;
            pair_slot[q] = (int32_t)slot;
        }
        ++slot;
    }
    if (!staged) return;   // uniform: `total` is the same in every lane
    __syncthreads();
    for (uint32_t e = lane; e < total; e += DIRECT_THREADS) {
        const uint32_t q = stage_q[e];
        pair_in[q] = stage_in[e];
        pair_slot[q] = stage_slot[e];
    }
}

size_t direct_notes_bytes(int64_t n) {
    return ptv3_align256((size_t)n * 8 * sizeof(uint32_t)) + ptv3_align256((size_t)n * 2 * sizeof(uint64_t));
}

DirectNotes carve_notes(void* base, int64_t n) {
    DirectNotes d;
    d.slot = (uint32_t*)base;
    d.found = (uint64_t*)((char*)base + ptv3_align256((size_t)n * 8 * sizeof(uint32_t)));
    return d;
}

size_t direct_plan_bytes(int64_t n, int taps) {
    return vh_bytes(n) + direct_notes_bytes(n) + carve_plan(nullptr, n, taps, DIRECT_THREADS).bytes;
}

// ---- the 3x3x3 pair lists of a voxel set from its 5x5x5 lists: the inner 27 taps of the 5x5x5
// neighbourhood ARE the 3x3x3 neighbourhood, so their tap-major segments are copied and only the
// output-major slots are renumbered (a stem with a 5x5x5 kernel and blocks with 3x3x3 kernels share
// level 0: one voxel hash and one neighbour search instead of two).
__device__ __forceinline__ int inner_tap5(int t3) {   // index among the 125 taps of 3x3x3 tap t3
    const int dx = t3 / 9, dy = (t3 / 3) % 3, dz = t3 % 3;
    return ((dx + 1) * 5 + (dy + 1)) * 5 + (dz + 1);
}

// thread = voxel: its 3x3x3 taps (bit t3) and their number, from the tap set the 5x5x5 count pass left
__global__ __launch_bounds__(PLAN_THREADS) void inner_count_kernel(DirectNotes notes, int64_t n,
                                                                   uint32_t* __restrict__ found3,
                                                                   int32_t* __restrict__ row_cnt3) {
    const int64_t i = (int64_t)blockIdx.x * PLAN_THREADS + threadIdx.x;
    if (i >= n) return;
    const uint64_t lo = notes.found[i], hi = notes.found[n + i];
    uint32_t f = 0;
#pragma unroll
    for (int t3 = 0; t3 < 27; ++t3) {
        const int t5 = inner_tap5(t3);
        const uint64_t bit = t5 < 64 ? (lo >> t5) & 1ull : (hi >> (t5 - 64)) & 1ull;
        f |= (uint32_t)bit << t3;
    }
    found3[i] = f;
    row_cnt3[i] = __popc(f);
}

// one work-group: tap_ptr3 = exclusive scan of the inner taps' counts, total to *n_pairs3
__global__ __launch_bounds__(64) void inner_tap_ptr_kernel(const int32_t* __restrict__ tap_ptr5,
                                                           int32_t* __restrict__ tap_ptr3,
                                                           int64_t* __restrict__ n_pairs3) {
    const int lane = threadIdx.x;
    int c = 0;
    if (lane < 27) {
        const int t5 = inner_tap5(lane);
        c = tap_ptr5[t5 + 1] - tap_ptr5[t5];
    }
    int x = c;
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) {
        const int y = __shfl_up(x, off, PTV3_WAVE);
        if (lane >= off) x += y;
    }
    if (lane < 27) tap_ptr3[lane] = x - c;
    if (lane == 26) {
        tap_ptr3[27] = x;
        *n_pairs3 = x;
    }
}

// thread = pair of the 3x3x3 lists: copy its input row, renumber its output slot
__global__ __launch_bounds__(PLAN_THREADS) void inner_fill_kernel(
    const int32_t* __restrict__ tap_ptr5, const int32_t* __restrict__ row_ptr5, const int32_t* __restrict__ pair_in5,
    const int32_t* __restrict__ pair_slot5, int64_t n, const uint32_t* __restrict__ found3,
    const int32_t* __restrict__ tap_ptr3, const int32_t* __restrict__ row_ptr3, int32_t* __restrict__ pair_in3,
    int32_t* __restrict__ pair_slot3) {
    __shared__ int32_t tp3[28], base5[27];
    if (threadIdx.x < 28) tp3[threadIdx.x] = tap_ptr3[threadIdx.x];
    if (threadIdx.x < 27) base5[threadIdx.x] = tap_ptr5[inner_tap5(threadIdx.x)];
    __syncthreads();
    const int64_t q3 = (int64_t)blockIdx.x * PLAN_THREADS + threadIdx.x;
    if (q3 >= tp3[27]) return;
    int lo = 0, hi = 27;   // the (non-empty) tap whose segment holds q3
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tp3[mid] <= (int32_t)q3) lo = mid; else hi = mid;
    }
    const int t3 = lo;
    const int64_t q5 = (int64_t)base5[t3] + (q3 - tp3[t3]);
    pair_in3[q3] = pair_in5[q5];
    // output voxel of the pair: the row whose 5x5x5 slot range holds its slot
    const int32_t slot5 = pair_slot5[q5];
    int64_t a = 0, b = n;   // largest i with row_ptr5[i] <= slot5
    while (b - a > 1) {
        const int64_t mid = (a + b) >> 1;
        if (row_ptr5[mid] <= slot5) a = mid; else b = mid;
    }
    pair_slot3[q3] = row_ptr3[a] + __popc(found3[a] & ((1u << t3) - 1u));
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
    hipLaunchKernelGGL(plan_scan_kernel, dim3((unsigned)(taps + 1)), dim3(SCAN_THREADS), 0, stream,
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

extern "C" size_t ptv3_kmap_plan_workspace_bytes(int64_t n, int ks) {
    if (n < 0 || (ks != 3 && ks != 5)) return 0;
    return direct_plan_bytes(n, ks * ks * ks);
}

extern "C" int ptv3_kmap_plan_count(const int32_t* indices, int64_t n, int ks, int32_t* tap_ptr, int64_t* n_pairs,
                                    void* workspace, size_t workspace_bytes, void* stream_) {
    if (n < 1 || n >= (1ll << 31) / 128) return PTV3_EINVAL;
    if (ks != 3 && ks != 5) return PTV3_ESHAPE;
    if (!indices || !tap_ptr || !n_pairs || !workspace) return PTV3_EINVAL;
    const int taps = ks * ks * ks;
    if (workspace_bytes < direct_plan_bytes(n, taps)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const VoxelHash h = vh_build(workspace, indices, n, stream);
    const DirectNotes notes = carve_notes((char*)workspace + vh_bytes(n), n);
    PlanWs w = carve_plan((char*)workspace + vh_bytes(n) + direct_notes_bytes(n), n, taps, DIRECT_THREADS);
    const int64_t blocks = ptv3_ceil_div(n, DIRECT_THREADS);
    if (ks == 3)
        hipLaunchKernelGGL(direct_count_kernel<3>, dim3((unsigned)blocks), dim3(DIRECT_THREADS), 0, stream, indices, n,
                           h, notes, w.row_cnt, w.blk_row_sum, w.blk_tap_cnt);
    else
        hipLaunchKernelGGL(direct_count_kernel<5>, dim3((unsigned)blocks), dim3(DIRECT_THREADS), 0, stream, indices, n,
                           h, notes, w.row_cnt, w.blk_row_sum, w.blk_tap_cnt);
    hipLaunchKernelGGL(plan_scan_kernel, dim3((unsigned)(taps + 1)), dim3(SCAN_THREADS), 0, stream,
                       w.blk_tap_cnt, w.blk_row_sum, blocks, taps, w.tap_total, n_pairs);
    hipLaunchKernelGGL(plan_tap_ptr_kernel, dim3(1), dim3(PLAN_THREADS), 0, stream,
                       (const uint32_t*)w.tap_total, taps, tap_ptr);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_kmap_plan_fill(const int32_t* indices, int64_t n, int ks, const int32_t* tap_ptr,
                                   int32_t* row_ptr, int32_t* pair_in, int32_t* pair_slot, void* workspace,
                                   size_t workspace_bytes, void* stream_) {
    if (n < 1 || n >= (1ll << 31) / 128) return PTV3_EINVAL;
    if (ks != 3 && ks != 5) return PTV3_ESHAPE;
    if (!indices || !tap_ptr || !row_ptr || !pair_in || !pair_slot || !workspace) return PTV3_EINVAL;
    const int taps = ks * ks * ks;
    if (workspace_bytes < direct_plan_bytes(n, taps)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const VoxelHash h = vh_view(workspace, n);   // built by ptv3_kmap_plan_count in this workspace
    const DirectNotes notes = carve_notes((char*)workspace + vh_bytes(n), n);
    PlanWs w = carve_plan((char*)workspace + vh_bytes(n) + direct_notes_bytes(n), n, taps, DIRECT_THREADS);
    const int64_t blocks = ptv3_ceil_div(n, DIRECT_THREADS);
    if (ks == 3)
        hipLaunchKernelGGL(direct_fill_kernel<3>, dim3((unsigned)blocks), dim3(DIRECT_THREADS), 0, stream, indices, n, h,
                           notes, (const uint32_t*)w.row_cnt, (const uint32_t*)w.blk_row_sum, (const uint32_t*)w.blk_tap_cnt,
                           tap_ptr, row_ptr, pair_in, pair_slot);
    else
        hipLaunchKernelGGL(direct_fill_kernel<5>, dim3((unsigned)blocks), dim3(DIRECT_THREADS), 0, stream, indices, n, h,
                           notes, (const uint32_t*)w.row_cnt, (const uint32_t*)w.blk_row_sum, (const uint32_t*)w.blk_tap_cnt,
                           tap_ptr, row_ptr, pair_in, pair_slot);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_kmap_plan_inner_count(const int32_t* tap_ptr5, int64_t n, const void* workspace5,
                                          size_t workspace5_bytes, int32_t* found3, int32_t* row_cnt3,
                                          int32_t* tap_ptr3, int64_t* n_pairs3, void* stream_) {
    if (n < 1 || n >= (1ll << 31) / 128) return PTV3_EINVAL;
    if (!tap_ptr5 || !workspace5 || !found3 || !row_cnt3 || !tap_ptr3 || !n_pairs3) return PTV3_EINVAL;
    if (workspace5_bytes < direct_plan_bytes(n, 125)) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const DirectNotes notes = carve_notes((char*)workspace5 + vh_bytes(n), n);   // left by ptv3_kmap_plan_count(ks = 5)
    hipLaunchKernelGGL(inner_count_kernel, dim3((unsigned)ptv3_ceil_div(n, PLAN_THREADS)), dim3(PLAN_THREADS), 0, stream,
                       notes, n, (uint32_t*)found3, row_cnt3);
    hipLaunchKernelGGL(inner_tap_ptr_kernel, dim3(1), dim3(64), 0, stream, tap_ptr5, tap_ptr3, n_pairs3);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_kmap_plan_inner_fill(const int32_t* tap_ptr5, const int32_t* row_ptr5, const int32_t* pair_in5,
                                         const int32_t* pair_slot5, int64_t n, int64_t n_pairs5, const int32_t* found3,
                                         const int32_t* tap_ptr3, const int32_t* row_ptr3, int32_t* pair_in3,
                                         int32_t* pair_slot3, void* stream_) {
    if (n < 1 || n_pairs5 < 1) return PTV3_EINVAL;
    if (!tap_ptr5 || !row_ptr5 || !pair_in5 || !pair_slot5 || !found3 || !tap_ptr3 || !row_ptr3 || !pair_in3 || !pair_slot3)
        return PTV3_EINVAL;
    // the 3x3x3 lists are at most as long as the 5x5x5 ones: threads past their end leave at once
    hipLaunchKernelGGL(inner_fill_kernel, dim3((unsigned)ptv3_ceil_div(n_pairs5, PLAN_THREADS)), dim3(PLAN_THREADS), 0,
                       (hipStream_t)stream_, tap_ptr5, row_ptr5, pair_in5, pair_slot5, n, (const uint32_t*)found3, tap_ptr3,
                       row_ptr3, pair_in3, pair_slot3);
    PTV3_RETURN_LAUNCH();
}
