// Backward kernels of the sparse operators around the attention: the weight gradient of the
// submanifold convolution and the gradient of the segment reductions of grid pooling.
//
// * spconv.SubMConv3d (call sites model.py:546-552, :767-774): for out[i] = sum_t W[:,t,:] x[nbr[i][t]]
//   the input gradient is the same convolution with the taps mirrored and the weight transposed
//   (nbr[i][t] = j  <=>  nbr[j][V-1-t] = i), which the forward kernels already compute; what is new
//   is   dW[co][t][ci] = sum_i dy[i][co] * x[nbr[i][t]][ci],   here per (tap, 64x64 weight block, range of
//   voxels). Half precision: the valid (voxel, neighbour) pairs of the range are compacted into LDS, each wave
//   takes 32 of them per step, writes both operands transposed into LDS (the MFMA wants the summed
//   index contiguous per lane) and accumulates up to 2x2 tiles of v_mfma_f32_32x32x16; fp32 atomics at
//   the end. fp32 and channel counts that are not multiples of 8: the same on plain FMAs, 4x4 sums per thread.
// * nn.Linear's weight gradient dW = dy^T x (the qkv / proj / fc1 / fc2 / cpe Linears, model.py:366-367,
//   :505-507, :553): the same kernel without the gather -- a reduction over several hundred thousand rows
//   into a weight of a few dozen channels, which a general GEMM handles badly.
// * nn.LayerNorm (model.py:554, :557, :572): with xhat = (x - mean) * rstd and g = dy * gamma,
//   dx = rstd * (g - mean(g) - xhat * mean(g * xhat)), dgamma = sum_rows dy * xhat, dbeta = sum_rows dy. Mean and
//   rstd are recomputed from x (two passes over the registers, like the forward kernel); 8 channels per
//   lane, a row per C / 8 lanes, column sums kept per lane over the rows and combined through LDS and
//   one atomic per work-group and channel. The training forward and backward kernels also take the
//   residual add in front of the LayerNorm (model.py:589-604) and its stochastic-depth factor, and read
//   and write every tensor in its own dtype (float residual stream, half-precision branches under autocast).
// * nn.BatchNorm1d in training mode, with the nn.GELU behind it (model.py:776-779, :707-710, :729-735): column
//   statistics over all rows (sums of x - pivot and of its square per lane, pivot = the first row, so that
//   a large mean does not cancel the variance), a one-work-group kernel that turns them into mean / rstd and
//   updates the running averages, the normalisation itself by the inference kernel with the batch
//   statistics; backward in two passes over x and dy: the column sums of dz and dz * xhat (dz = dy *
//   gelu'(z), z recomputed), then dx = gamma * rstd * (dz - mean(dz) - xhat * mean(dz * xhat)).
// * torch_scatter.segment_csr (model.py:684-689): max / min send the gradient of a cluster to the first
//   member that attains the value, sum copies it to every member, mean divides it by the cluster size.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// ---- d[m][tap][k] += sum over rows of a[row][m] * b[src(row)][k] on the matrix cores.
// A work-group covers a 64 x 64 block of d and a range of rows; each of its four waves takes 32 rows per
// step: 16-byte pieces of the two operands are written transposed into the wave's LDS tiles (rows of
// OR_S halves, 16-byte chunks swizzled by the channel group so that the writes spread over the banks),
// then read back as MFMA operands.
constexpr int XCDS = 8;   // work-groups of a launch go to the XCDs round-robin; each XCD has an L2 of its own

// Which (tap, range of rows, block of the result) this work-group takes. All blocks of one (tap, range) read the
// same rows, so they should meet in one L2: they are dealt to the same XCD, next to each other, while the (tap,
// range) pairs themselves stay interleaved over the XCDs in launch order (with one block per range this is the
// plain order; handing each XCD a contiguous eighth of the pairs measured 25 % slower on the gathering form).
// The grid is ceil(taps * splits / 8) * 8 * blocks work-groups; the ones past the last pair leave.
template <int SIDE>
__device__ __forceinline__ bool outer_item(int taps, int splits, int m_total, int k_total, int* tap, int* split, int* m0,
                                           int* k0) {
    const int bm = (m_total + SIDE - 1) / SIDE, bk = (k_total + SIDE - 1) / SIDE;
    const int slot = blockIdx.x / XCDS;
    const int64_t x = (int64_t)(slot / (bm * bk)) * XCDS + blockIdx.x % XCDS;
    if (x >= (int64_t)taps * splits) return false;
    const int blk = slot % (bm * bk);
    *tap = (int)(x / splits);
    *split = (int)(x % splits);
    *m0 = (blk % bm) * SIDE;
    *k0 = (blk / bm) * SIDE;
    return true;
}

constexpr int OR_S = 40;      // halves per LDS row: 32 summed rows + padding that spreads the operand reads
constexpr int OR_C = 64;      // channels per block side
constexpr int OR_LIST = 4096; // most rows per work-group with GATHER (the compacted pair list lives in LDS)

template <typename T> struct Mfma16;
template <> struct Mfma16<_Float16> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<__bf16> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

// writes pieces of four consecutive rows 4 q .. 4 q + 3 (8 channels of group g each) transposed: per channel the
// four halves are one 8-byte word at tile[8 g + c][4 q], chunks of 8 rows swizzled by the channel group
__device__ __forceinline__ void put_transposed4(uint16_t* tile, int g, int q, const u32x4* w) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    uint16_t* base = tile + (8 * g) * OR_S + (((q >> 1) ^ (g & 3)) << 3) + ((q & 1) << 2);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        // words w[j][p] hold channels (2 p, 2 p + 1) of row j
        const u32x2 even = {__builtin_amdgcn_perm(w[1][p], w[0][p], 0x05040100u), __builtin_amdgcn_perm(w[3][p], w[2][p], 0x05040100u)};
        const u32x2 odd = {__builtin_amdgcn_perm(w[1][p], w[0][p], 0x07060302u), __builtin_amdgcn_perm(w[3][p], w[2][p], 0x07060302u)};
        *(u32x2*)(base + (2 * p) * OR_S) = even;
        *(u32x2*)(base + (2 * p + 1) * OR_S) = odd;
    }
}

template <typename T, bool GATHER>
__global__ __launch_bounds__(256) void outer_rows_kernel(const T* __restrict__ a, const T* __restrict__ b, int64_t n,
                                                         int m_total, int k_total, const int32_t* __restrict__ nbr,
                                                         const int32_t* __restrict__ tap_ptr,
                                                         const int32_t* __restrict__ pair_in,
                                                         int taps, int splits, int64_t rows_per_split,
                                                         int64_t slab_stride, float* __restrict__ d,
                                                         float* __restrict__ colsum) {
    typedef typename Mfma16<T>::v8 v8;
    __shared__ float wave_cols[4][OR_C];
    __shared__ __align__(16) uint16_t tiles[4][2][OR_C * OR_S];
    __shared__ int32_t list_a[GATHER ? OR_LIST : 1], list_b[GATHER ? OR_LIST : 1];
    __shared__ int list_n;
    int tap, split, m0, k0;
    if (!outer_item<OR_C>(taps, splits, m_total, k_total, &tap, &split, &m0, &k0)) return;
    const int tm = min(2, (m_total - m0 + 31) / 32), tk = min(2, (k_total - k0 + 31) / 32);
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    int64_t r0 = (int64_t)split * rows_per_split;
    const int64_t r1 = min(n, r0 + rows_per_split);
    int count = (int)(r1 - r0);
    if (GATHER && tap_ptr) {
        // the tap's own list of (output row, input row) pairs, rows_per_split of them per range: nbr holds the
        // output rows here.
        const int64_t p0 = tap_ptr[tap] + (int64_t)split * rows_per_split;
        const int64_t left = (int64_t)tap_ptr[tap + 1] - p0;
        count = left < 0 ? 0 : (int)min(left, rows_per_split);
        // past the end of a short tap's list: the sum over ranges skips this one (a single range is the result itself)
        if (count == 0 && splits > 1) return;
        for (int e = tid; e < count; e += 256) {
            list_a[e] = nbr[p0 + e];
            list_b[e] = pair_in[p0 + e];
        }
        r0 = 0;
        __syncthreads();
    } else if (GATHER) {
        // compact the voxels of the range that have this neighbour: (output row, input row) pairs
        if (tid == 0) list_n = 0;
        __syncthreads();
        const int32_t* nb = nbr + (int64_t)tap * n;
        for (int64_t e = r0 + tid; e < r0 + ((r1 - r0 + 255) / 256) * 256; e += 256) {
            const int32_t src = e < r1 ? nb[e] : -1;
            const uint64_t mask = __ballot(src >= 0);
            int base = 0;
            if (lane == 0 && mask) base = atomicAdd(&list_n, __popcll(mask));
            base = __shfl(base, 0, PTV3_WAVE);
            if (src >= 0) {
                const int pos = base + __popcll(mask & ((1ull << lane) - 1));
                list_a[pos] = (int32_t)(e - r0);
                list_b[pos] = src;
            }
        }
        __syncthreads();
        count = list_n;
    }
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    uint16_t* ta = tiles[wave][0];
    uint16_t* tb = tiles[wave][1];
    const int g = lane & 7, rq = lane >> 3;   // pieces: channel group g, rows 4 rq + j
    const bool a_in = m0 + 8 * g < m_total, b_in = k0 + 8 * g < k_total;
    const int col = lane & 31, hf = lane >> 5;
    // column sums of a (the bias gradient) ride along in the blocks that read each of a's rows exactly once:
    // the first block along k, and with GATHER the centre tap, whose pairs are (i, i) for every voxel
    const bool sum_cols = colsum != nullptr && k0 == 0 && (!GATHER || tap == taps / 2);
    float cs[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) cs[c] = 0.f;
    // A wave's LDS tiles are its own and its LDS operations complete in order, so the loop needs no barrier:
    // the waves drift apart and hide each other's load latency. The pieces of the next step are requested as
    // soon as this step's have been written to LDS, and arrive while the MFMAs run.
    u32x4 wa[4], wb[4];
    auto fetch = [&](int base) {
        const int mine = base + wave * 32;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int idx = mine + 4 * rq + j;
            wa[j] = (u32x4){0, 0, 0, 0};
            wb[j] = (u32x4){0, 0, 0, 0};
            if (idx < count) {
                const int64_t ra = r0 + (GATHER ? list_a[idx] : idx);
                const int64_t rb = GATHER ? (int64_t)list_b[idx] : ra;
                if (a_in) wa[j] = *(const u32x4*)(a + ra * m_total + m0 + 8 * g);
                if (b_in) wb[j] = *(const u32x4*)(b + rb * k_total + k0 + 8 * g);
            }
        }
    };
    if (count > 0) fetch(0);
    for (int base = 0; base < count; base += 4 * 32) {
        if (sum_cols) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v8 h = __builtin_bit_cast(v8, wa[j]);
#pragma unroll
                for (int c = 0; c < 8; ++c) cs[c] += (float)h[c];
            }
        }
        put_transposed4(ta, g, rq, wa);
        put_transposed4(tb, g, rq, wb);
        if (base + 4 * 32 < count) fetch(base + 4 * 32);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int ch = 32 * i + col;
                const int chunk = (2 * ks + hf) ^ ((ch >> 3) & 3);
                fa[i] = __builtin_bit_cast(v8, *(const u32x4*)(ta + ch * OR_S + 8 * chunk));
                fb[i] = __builtin_bit_cast(v8, *(const u32x4*)(tb + ch * OR_S + 8 * chunk));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (i < tm && j < tk) acc[i][j] = Mfma16<T>::mfma(fa[i], fb[j], acc[i][j]);
        }
    }
    __syncthreads();   // every wave is done with its tiles
    // the four waves hold sums over different rows: add them up in LDS (the operand tiles are free now), then
    // every thread stores 16 of the block's 64 x 64 values into this split's slab, without atomics.
    // acc[i][j][v]: m = 32 i + 8 (v / 4) + 4 hf + v % 4, k = 32 j + col
    float* sum = (float*)&tiles[0][0][0];   // 64 x 64 floats = 16 KB of the 40 KB
    for (int w = 0; w < 4; ++w) {
        if (wave == w) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        float* at = sum + (32 * i + 8 * (v >> 2) + 4 * hf + (v & 3)) * OR_C + 32 * j + col;
                        *at = (w == 0 ? 0.f : *at) + acc[i][j][v];
                    }
        }
        __syncthreads();
    }
    float* slab = d + (int64_t)split * slab_stride;
    for (int e = tid; e < OR_C * OR_C; e += 256) {
        const int m = m0 + e / OR_C, k = k0 + e % OR_C;
        if (m < m_total && k < k_total) slab[((int64_t)m * taps + tap) * k_total + k] = sum[e];
    }
    if (sum_cols) {   // the same for the whole work-group
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            cs[c] += __shfl_xor(cs[c], 8, PTV3_WAVE);
            cs[c] += __shfl_xor(cs[c], 16, PTV3_WAVE);
            cs[c] += __shfl_xor(cs[c], 32, PTV3_WAVE);
        }
        if (rq == 0) {
#pragma unroll
            for (int c = 0; c < 8; ++c) wave_cols[wave][8 * g + c] = cs[c];
        }
        __syncthreads();
        if (tid < OR_C && m0 + tid < m_total)
            colsum[(int64_t)split * slab_stride + m0 + tid] =
                wave_cols[0][tid] + wave_cols[1][tid] + wave_cols[2][tid] + wave_cols[3][tid];
    }
}

// The same reduction for results of 128 channels or more a side: a work-group owns a 128 x 128 block, its
// four waves a 64 x 64 quadrant each, and the 32 rows of a step are staged once for all of them (threads
// 0..127 the pieces of a, 128..255 those of b) into one of two LDS buffers, a barrier per step. Per MFMA that
// is half the operand traffic and half the staging work of the 64 x 64 form, which at 256 channels is bound by
// the gathered 128-byte pieces coming out of L2.
constexpr int OW_C = 128;

template <typename T, bool GATHER>
__global__ __launch_bounds__(256) void outer_rows_wide_kernel(const T* __restrict__ a, const T* __restrict__ b, int64_t n,
                                                              int m_total, int k_total, const int32_t* __restrict__ nbr,
                                                              const int32_t* __restrict__ tap_ptr,
                                                              const int32_t* __restrict__ pair_in,
                                                              int taps, int splits, int64_t rows_per_split,
                                                              int64_t slab_stride, float* __restrict__ d,
                                                              float* __restrict__ colsum) {
    typedef typename Mfma16<T>::v8 v8;
    __shared__ __align__(16) uint16_t tiles[2][2][OW_C * OR_S];
    __shared__ int32_t list_a[GATHER ? OR_LIST : 1], list_b[GATHER ? OR_LIST : 1];
    __shared__ int list_n;
    __shared__ float wave_cols[2][OW_C];
    int tap, split, m0, k0;
    if (!outer_item<OW_C>(taps, splits, m_total, k_total, &tap, &split, &m0, &k0)) return;
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    int64_t r0 = (int64_t)split * rows_per_split;
    const int64_t r1 = min(n, r0 + rows_per_split);
    int count = (int)(r1 - r0);
    if (GATHER && tap_ptr) {
        // the tap's own list of (output row, input row) pairs, rows_per_split of them per range: nbr holds the
        // output rows here.
        const int64_t p0 = tap_ptr[tap] + (int64_t)split * rows_per_split;
        const int64_t left = (int64_t)tap_ptr[tap + 1] - p0;
        count = left < 0 ? 0 : (int)min(left, rows_per_split);
        // past the end of a short tap's list: the sum over ranges skips this one (a single range is the result itself)
        if (count == 0 && splits > 1) return;
        for (int e = tid; e < count; e += 256) {
            list_a[e] = nbr[p0 + e];
            list_b[e] = pair_in[p0 + e];
        }
        r0 = 0;
        __syncthreads();
    } else if (GATHER) {
        if (tid == 0) list_n = 0;
        __syncthreads();
        const int32_t* nb = nbr + (int64_t)tap * n;
        for (int64_t e = r0 + tid; e < r0 + ((r1 - r0 + 255) / 256) * 256; e += 256) {
            const int32_t src = e < r1 ? nb[e] : -1;
            const uint64_t mask = __ballot(src >= 0);
            int base = 0;
            if (lane == 0 && mask) base = atomicAdd(&list_n, __popcll(mask));
            base = __shfl(base, 0, PTV3_WAVE);
            if (src >= 0) {
                const int pos = base + __popcll(mask & ((1ull << lane) - 1));
                list_a[pos] = (int32_t)(e - r0);
                list_b[pos] = src;
            }
        }
        __syncthreads();
        count = list_n;
    }
    // this wave's quadrant, 2 x 2 tiles
    const int qm = (wave & 1) * 64, qk = (wave >> 1) * 64;
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    // staging role: operand, channel group, row quad
    const bool is_b = tid >= 128;
    const int st = tid & 127, g = st & 15, rq = st >> 4;
    const T* src_ptr = is_b ? b : a;
    const int width = is_b ? k_total : m_total, c0 = (is_b ? k0 : m0) + 8 * g;
    const bool in_range = c0 < width;
    const bool sum_cols = colsum != nullptr && k0 == 0 && (!GATHER || tap == taps / 2);
    float cs[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) cs[c] = 0.f;
    u32x4 w[4];
    auto fetch = [&](int base) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int idx = base + 4 * rq + j;
            w[j] = (u32x4){0, 0, 0, 0};
            if (idx < count && in_range) {
                const int64_t ra = r0 + (GATHER ? list_a[idx] : idx);
                const int64_t row = is_b ? (GATHER ? (int64_t)list_b[idx] : ra) : ra;
                w[j] = *(const u32x4*)(src_ptr + row * width + c0);
            }
        }
    };
    const int col = lane & 31, hf = lane >> 5;
    if (count > 0) fetch(0);
    int buf = 0;
    for (int base = 0; base < count; base += 32, buf ^= 1) {
        if (sum_cols && !is_b) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v8 h = __builtin_bit_cast(v8, w[j]);
#pragma unroll
                for (int c = 0; c < 8; ++c) cs[c] += (float)h[c];
            }
        }
        put_transposed4(tiles[buf][is_b], g, rq, w);
        if (base + 32 < count) fetch(base + 32);
        // One barrier per step: it also keeps a wave from overwriting this buffer two steps on while another
        // still reads it, because nobody passes the next step's barrier before everyone has finished these reads.
        __syncthreads();
        const uint16_t* ta = tiles[buf][0];
        const uint16_t* tb = tiles[buf][1];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int cha = qm + 32 * i + col, chb = qk + 32 * i + col;
                fa[i] = __builtin_bit_cast(v8, *(const u32x4*)(ta + cha * OR_S + 8 * ((2 * ks + hf) ^ ((cha >> 3) & 3))));
                fb[i] = __builtin_bit_cast(v8, *(const u32x4*)(tb + chb * OR_S + 8 * ((2 * ks + hf) ^ ((chb >> 3) & 3))));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = Mfma16<T>::mfma(fa[i], fb[j], acc[i][j]);
        }
    }
    // acc[i][j][v]: m = m0 + qm + 32 i + 8 (v / 4) + 4 hf + v % 4, k = k0 + qk + 32 j + col; the quadrant is this wave's alone
    float* slab = d + (int64_t)split * slab_stride;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int k = k0 + qk + 32 * j + col;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + qm + 32 * i + 8 * (v >> 2) + 4 * hf + (v & 3);
                if (m < m_total && k < k_total) slab[((int64_t)m * taps + tap) * k_total + k] = acc[i][j][v];
            }
        }
    if (sum_cols) {   // the same for the whole work-group; waves 0 and 1 staged a
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            cs[c] += __shfl_xor(cs[c], 16, PTV3_WAVE);
            cs[c] += __shfl_xor(cs[c], 32, PTV3_WAVE);
        }
        if (!is_b && lane < 16) {
#pragma unroll
            for (int c = 0; c < 8; ++c) wave_cols[wave][8 * g + c] = cs[c];
        }
        __syncthreads();
        if (tid < OW_C && m0 + tid < m_total)
            colsum[(int64_t)split * slab_stride + m0 + tid] = wave_cols[0][tid] + wave_cols[1][tid];
    }
}

// out[i] = sum over the splits' slabs (of `stride` floats, the first `total` of them summed): a work-group takes 32 neighbouring values, its 8 thread rows share
// out the splits (four loads in flight each) and meet in LDS
// With tap_ptr (pair-list ranges) the value i = (m * taps + tap) * k_total + k of the first result only has the
// ranges its tap's list reaches: ceil(pairs of the tap / rows_per_split) of them; the others were never written.
__global__ __launch_bounds__(256) void slab_sum_kernel(const float* __restrict__ slabs, int64_t stride, int64_t total,
                                                       int splits, float* __restrict__ out, int64_t first,
                                                       float* __restrict__ out2, const int32_t* __restrict__ tap_ptr,
                                                       int taps, int k_total, int64_t rows_per_split) {
    __shared__ float part[8][32];
    const int e = threadIdx.x % 32, lane_s = threadIdx.x / 32;
    const int64_t i = (int64_t)blockIdx.x * 32 + e;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
    if (i < total) {
        if (tap_ptr && i < first) {
            const int t = (int)(((uint32_t)i / (uint32_t)k_total) % (uint32_t)taps);   // first < 2^31: checked at launch
            const int64_t have = ((int64_t)tap_ptr[t + 1] - tap_ptr[t] + rows_per_split - 1) / rows_per_split;
            if (have < splits) splits = (int)have;
        }
        int s = lane_s;
        for (; s + 24 < splits; s += 32) {
            v0 += slabs[(int64_t)s * stride + i];
            v1 += slabs[(int64_t)(s + 8) * stride + i];
            v2 += slabs[(int64_t)(s + 16) * stride + i];
            v3 += slabs[(int64_t)(s + 24) * stride + i];
        }
        for (; s < splits; s += 8) v0 += slabs[(int64_t)s * stride + i];
    }
    part[lane_s][e] = (v0 + v1) + (v2 + v3);
    __syncthreads();
    if (lane_s == 0 && i < total) {
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) v += part[k][e];
        if (i < first) out[i] = v; else out2[i - first] = v;   // a slab's tail goes to the second result
    }
}

__global__ __launch_bounds__(256) void zero_kernel(float* __restrict__ out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) out[i] = 0.f;
}

template <typename T> struct Row8;
template <> struct Row8<float> {
    static __device__ __forceinline__ void load(const float* p, float* v) {
        const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    static __device__ __forceinline__ void store(float* p, const float* v) {
        *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
        *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};
template <typename H> struct Row8Half {
    typedef H h8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ void load(const H* p, float* v) {
        const h8 a = *(const h8*)p;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)a[i];
    }
    static __device__ __forceinline__ void store(H* p, const float* v) {
        h8 a;
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = (H)v[i];
        *(h8*)p = a;
    }
};
template <> struct Row8<_Float16> : Row8Half<_Float16> {};
template <> struct Row8<__bf16> : Row8Half<__bf16> {};

template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
    for (int off = 1; off < LPR; off <<= 1) v += __shfl_xor(v, off, PTV3_WAVE);
    return v;
}

// 8 consecutive values in any of the three dtypes, as floats
__device__ __forceinline__ void load8_any(const void* p, int dtype, int64_t off, float* v) {
    if (dtype == PTV3_F32) Row8<float>::load((const float*)p + off, v);
    else if (dtype == PTV3_F16) Row8<_Float16>::load((const _Float16*)p + off, v);
    else Row8<__bf16>::load((const __bf16*)p + off, v);
}
__device__ __forceinline__ void store8_any(void* p, int dtype, int64_t off, const float* v) {
    if (dtype == PTV3_F32) Row8<float>::store((float*)p + off, v);
    else if (dtype == PTV3_F16) Row8<_Float16>::store((_Float16*)p + off, v);
    else Row8<__bf16>::store((__bf16*)p + off, v);
}
__device__ __forceinline__ float load1_any(const void* p, int dtype, int64_t off) {
    if (dtype == PTV3_F32) return ((const float*)p)[off];
    if (dtype == PTV3_F16) return (float)((const _Float16*)p)[off];
    return (float)((const __bf16*)p)[off];
}
__device__ __forceinline__ float round_any(float v, int dtype) {
    if (dtype == PTV3_F32) return v;
    if (dtype == PTV3_F16) return (float)(_Float16)v;
    return (float)(__bf16)v;
}

// The bits of 8 consecutive values, fetched without looking at them, and their conversion afterwards: a kernel
// issues the loads of all its operands back to back and converts once they have arrived (a conversion inside
// the dtype branch would make every load wait for the one before).
struct Raw8 {
    u32x4 lo, hi;
};
__device__ __forceinline__ Raw8 raw8_load(const void* p, int dtype, int64_t off) {
    Raw8 r;
    const char* b = (const char*)p + off * (dtype == PTV3_F32 ? 4 : 2);
    r.lo = *(const u32x4*)b;
    r.hi = (u32x4){0, 0, 0, 0};
    if (dtype == PTV3_F32) r.hi = *(const u32x4*)(b + 16);
    return r;
}
__device__ __forceinline__ void raw8_floats(const Raw8& r, int dtype, float* v) {
    if (dtype == PTV3_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t a = r.lo[i], b = r.hi[i];   // through scalars: a bit_cast of the subscript itself reads element 0
            v[i] = __builtin_bit_cast(float, a);
            v[4 + i] = __builtin_bit_cast(float, b);
        }
    } else if (dtype == PTV3_F16) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 h = __builtin_bit_cast(h8, r.lo);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)h[i];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __builtin_bit_cast(float, r.lo[i] << 16);
            v[2 * i + 1] = __builtin_bit_cast(float, r.lo[i] & 0xffff0000u);
        }
    }
}

// Tensors of one call, each with its own dtype: autocast mixes a float residual stream with half-precision
// branches, and the kernels read and write each in place instead of going through cast passes.
struct AnyRows {
    const void* p;
    int dtype;
};
struct AnyRowsOut {
    void* p;
    int dtype;
};

// sum = skip + branch * row_scale (skip and row_scale optional), y = LayerNorm(sum): 8 channels per lane, a row
// per LPR lanes; the statistics are taken from the sum as stored, so the backward kernel sees the same numbers.
// PRE: the branch goes through a LayerNorm of its own first (pre_gamma, pre_beta, pre_eps): the xCPE's norm in front
// of the first residual connection of a Block (model.py:546-554, :589-592).
template <int LPR, bool PRE>
__global__ __launch_bounds__(256) void add_layer_norm_fwd_kernel(AnyRows skip, AnyRows branch, AnyRows row_scale,
                                                                 AnyRows gamma, AnyRows beta, int64_t n, float eps,
                                                                 AnyRowsOut sum, AnyRowsOut y, AnyRows pre_gamma,
                                                                 AnyRows pre_beta, float pre_eps) {
    constexpr int C = LPR * 8, RPW = PTV3_WAVE / LPR;
    const int wave = threadIdx.x / PTV3_WAVE, lane = threadIdx.x % PTV3_WAVE;
    const int sub = lane % LPR, rsub = lane / LPR;
    float g[8], b[8], pg[8], pb[8];
    load8_any(gamma.p, gamma.dtype, sub * 8, g);
    load8_any(beta.p, beta.dtype, sub * 8, b);
    if (PRE) {
        load8_any(pre_gamma.p, pre_gamma.dtype, sub * 8, pg);
        load8_any(pre_beta.p, pre_beta.dtype, sub * 8, pb);
    }
    const int64_t stride = (int64_t)gridDim.x * 4 * RPW;
    for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW; row0 < n; row0 += stride) {
        const int64_t row = row0 + rsub;
        const bool valid = row < n;
        const int64_t off = row * C + sub * 8;
        float xv[8], sv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { xv[i] = 0.f; sv[i] = 0.f; }
        float m = 1.f;
        if (valid) {
            const Raw8 rb = raw8_load(branch.p, branch.dtype, off);
            Raw8 rs = rb;
            if (skip.p) rs = raw8_load(skip.p, skip.dtype, off);
            if (row_scale.p) m = load1_any(row_scale.p, row_scale.dtype, row);
            raw8_floats(rb, branch.dtype, xv);
            if (skip.p) raw8_floats(rs, skip.dtype, sv);
        }
        if (PRE) {   // every lane takes part in the row sums, rows past the end with zeros
            float ps = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ps += xv[i];
            const float pmean = row_sum<LPR>(ps) * (1.f / C);
            float pq = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { xv[i] -= pmean; pq = fmaf(xv[i], xv[i], pq); }
            const float prstd = rsqrtf(row_sum<LPR>(pq) * (1.f / C) + pre_eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = fmaf(xv[i] * prstd, pg[i], pb[i]);
        }
        if (valid) {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = fmaf(xv[i], m, sv[i]);
            if (sum.p) {
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[i] = round_any(xv[i], sum.dtype);
                store8_any(sum.p, sum.dtype, off, xv);
            }
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) s += xv[i];
        const float mean = row_sum<LPR>(s) * (1.f / C);
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) { xv[i] -= mean; q = fmaf(xv[i], xv[i], q); }
        const float rstd = rsqrtf(row_sum<LPR>(q) * (1.f / C) + eps);
        if (valid) {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = fmaf(xv[i] * rstd, g[i], b[i]);
            store8_any(y.p, y.dtype, off, xv);
        }
    }
}

// g = LayerNorm'(sum, dy) + dsum (dsum optional); dskip = g, dbranch = g * row_scale, each optional and in its
// own dtype; dgamma / dbeta accumulated in fp32. Mean and rstd are recomputed from sum.
// PRE: the branch came out of a LayerNorm of its own (see the forward kernel): pre_x is that norm's input,
// dbranch its gradient, dpre_gamma / dpre_beta the norm's parameter gradients.
template <int LPR, bool PRE>
__global__ __launch_bounds__(256) void add_layer_norm_bwd_kernel(AnyRows sum, AnyRows dy, AnyRows dsum, AnyRows row_scale,
                                                                 AnyRows gamma, int64_t n, float eps, AnyRowsOut dskip,
                                                                 AnyRowsOut dbranch, float* __restrict__ dgamma,
                                                                 float* __restrict__ dbeta, AnyRows pre_x,
                                                                 AnyRows pre_gamma, float pre_eps,
                                                                 float* __restrict__ dpre_gamma,
                                                                 float* __restrict__ dpre_beta) {
    constexpr int C = LPR * 8, RPW = PTV3_WAVE / LPR;
    __shared__ float part[PRE ? 4 : 2][4][C];
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int sub = lane % LPR, rsub = lane / LPR;
    float g[8], ag[8], ab[8], pg[8], pag[8], pab[8];
    load8_any(gamma.p, gamma.dtype, sub * 8, g);
    if (PRE) load8_any(pre_gamma.p, pre_gamma.dtype, sub * 8, pg);
#pragma unroll
    for (int i = 0; i < 8; ++i) { ag[i] = 0.f; ab[i] = 0.f; pag[i] = 0.f; pab[i] = 0.f; }
    const int64_t stride = (int64_t)gridDim.x * 4 * RPW;
    for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW; row0 < n; row0 += stride) {
        const int64_t row = row0 + rsub;
        const bool valid = row < n;
        const int64_t off = row * C + sub * 8;
        float xv[8], gv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { xv[i] = 0.f; gv[i] = 0.f; }
        float extra[8], scale = 1.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) extra[i] = 0.f;
        if (valid) {
            const Raw8 rx = raw8_load(sum.p, sum.dtype, off);
            const Raw8 rg = raw8_load(dy.p, dy.dtype, off);
            Raw8 re = rx;
            if (dsum.p) re = raw8_load(dsum.p, dsum.dtype, off);   // gradient arriving at the sum by another path
            if (row_scale.p && dbranch.p) scale = load1_any(row_scale.p, row_scale.dtype, row);
            raw8_floats(rx, sum.dtype, xv);
            raw8_floats(rg, dy.dtype, gv);
            if (dsum.p) raw8_floats(re, dsum.dtype, extra);
        }
        float cv[8];   // PRE: the input of the branch's own norm
#pragma unroll
        for (int i = 0; i < 8; ++i) cv[i] = 0.f;
        if (PRE && valid) {
            const Raw8 rc = raw8_load(pre_x.p, pre_x.dtype, off);
            raw8_floats(rc, pre_x.dtype, cv);
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) s += xv[i];
        const float mean = row_sum<LPR>(s) * (1.f / C);
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) { xv[i] -= mean; q = fmaf(xv[i], xv[i], q); }
        const float rstd = rsqrtf(row_sum<LPR>(q) * (1.f / C) + eps);
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            xv[i] *= rstd;                      // xhat
            ag[i] = fmaf(gv[i], xv[i], ag[i]);  // rows beyond n carry zeros
            ab[i] += gv[i];
            gv[i] *= g[i];
            s1 += gv[i];
            s2 = fmaf(gv[i], xv[i], s2);
        }
        s1 = row_sum<LPR>(s1) * (1.f / C);
        s2 = row_sum<LPR>(s2) * (1.f / C);
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = valid ? rstd * (gv[i] - s1 - xv[i] * s2) + extra[i] : 0.f;
        if (valid && dskip.p) store8_any(dskip.p, dskip.dtype, off, o);
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] *= scale;   // the gradient of the branch as it was added
        if (PRE) {
            // back through the branch's own norm: statistics again from its input, rows past the end carry zeros
            float cs = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) cs += cv[i];
            const float cmean = row_sum<LPR>(cs) * (1.f / C);
            float cq = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { cv[i] -= cmean; cq = fmaf(cv[i], cv[i], cq); }
            const float crstd = rsqrtf(row_sum<LPR>(cq) * (1.f / C) + pre_eps);
            float t1 = 0.f, t2 = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                cv[i] *= crstd;                        // xhat of the branch's norm
                pag[i] = fmaf(o[i], cv[i], pag[i]);
                pab[i] += o[i];
                o[i] *= pg[i];
                t1 += o[i];
                t2 = fmaf(o[i], cv[i], t2);
            }
            t1 = row_sum<LPR>(t1) * (1.f / C);
            t2 = row_sum<LPR>(t2) * (1.f / C);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = crstd * (o[i] - t1 - cv[i] * t2);
        }
        if (valid && dbranch.p) store8_any(dbranch.p, dbranch.dtype, off, o);
    }
    // column sums: over the rows a wave holds side by side, then over the waves, then one atomic per channel
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int off = LPR; off < PTV3_WAVE; off <<= 1) {
            ag[i] += __shfl_xor(ag[i], off, PTV3_WAVE);
            ab[i] += __shfl_xor(ab[i], off, PTV3_WAVE);
        }
    }
    if (PRE) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int off = LPR; off < PTV3_WAVE; off <<= 1) {
                pag[i] += __shfl_xor(pag[i], off, PTV3_WAVE);
                pab[i] += __shfl_xor(pab[i], off, PTV3_WAVE);
            }
        }
    }
    if (rsub == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            part[0][wave][sub * 8 + i] = ag[i];
            part[1][wave][sub * 8 + i] = ab[i];
            if (PRE) {
                part[2][wave][sub * 8 + i] = pag[i];
                part[3][wave][sub * 8 + i] = pab[i];
            }
        }
    }
    __syncthreads();
    for (int c = tid; c < (PRE ? 4 : 2) * C; c += 256) {
        const int which = c / C, ch = c % C;
        const float v = part[which][0][ch] + part[which][1][ch] + part[which][2][ch] + part[which][3][ch];
        float* dst = which == 0 ? dgamma : which == 1 ? dbeta : which == 2 ? dpre_gamma : dpre_beta;
        atomicAdd(dst + ch, v);
    }
}

int64_t ln_grid(int64_t n, int c) {
    const int64_t cap = 512;   // two work-groups per CU: more only add atomics on the column sums (measured)
    const int64_t rows_per_wg = 4 * (PTV3_WAVE / (c / 8));
    const int64_t grid = ptv3_ceil_div(n, rows_per_wg);
    return grid > cap ? cap : grid;
}

int launch_add_ln_fwd(AnyRows skip, AnyRows branch, AnyRows row_scale, AnyRows gamma, AnyRows beta, int64_t n, int c,
                      float eps, AnyRowsOut sum, AnyRowsOut y, AnyRows pre_gamma, AnyRows pre_beta, float pre_eps,
                      hipStream_t stream) {
#define PTV3_LNF(L)                                                                                                   \
    if (c == 8 * L) {                                                                                                 \
        if (pre_gamma.p)                                                                                              \
            hipLaunchKernelGGL((add_layer_norm_fwd_kernel<L, true>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0,     \
                               stream, skip, branch, row_scale, gamma, beta, n, eps, sum, y, pre_gamma, pre_beta,     \
                               pre_eps);                                                                              \
        else                                                                                                          \
            hipLaunchKernelGGL((add_layer_norm_fwd_kernel<L, false>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0,    \
                               stream, skip, branch, row_scale, gamma, beta, n, eps, sum, y, pre_gamma, pre_beta,     \
                               pre_eps);                                                                              \
        PTV3_RETURN_LAUNCH();                                                                                         \
    }
    PTV3_LNF(4) PTV3_LNF(8) PTV3_LNF(16) PTV3_LNF(32) PTV3_LNF(64)
#undef PTV3_LNF
    return PTV3_ESHAPE;
}

int launch_add_ln_bwd(AnyRows sum, AnyRows dy, AnyRows dsum, AnyRows row_scale, AnyRows gamma, int64_t n, int c, float eps,
                      AnyRowsOut dskip, AnyRowsOut dbranch, float* dgamma, float* dbeta, AnyRows pre_x, AnyRows pre_gamma,
                      float pre_eps, float* dpre_gamma, float* dpre_beta, hipStream_t stream) {
#define PTV3_LNB(L)                                                                                                   \
    if (c == 8 * L) {                                                                                                 \
        if (pre_x.p)                                                                                                  \
            hipLaunchKernelGGL((add_layer_norm_bwd_kernel<L, true>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0,     \
                               stream, sum, dy, dsum, row_scale, gamma, n, eps, dskip, dbranch, dgamma, dbeta, pre_x, \
                               pre_gamma, pre_eps, dpre_gamma, dpre_beta);                                            \
        else                                                                                                          \
            hipLaunchKernelGGL((add_layer_norm_bwd_kernel<L, false>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0,    \
                               stream, sum, dy, dsum, row_scale, gamma, n, eps, dskip, dbranch, dgamma, dbeta, pre_x, \
                               pre_gamma, pre_eps, dpre_gamma, dpre_beta);                                            \
        PTV3_RETURN_LAUNCH();                                                                                         \
    }
    PTV3_LNB(4) PTV3_LNB(8) PTV3_LNB(16) PTV3_LNB(32) PTV3_LNB(64)
#undef PTV3_LNB
    return PTV3_ESHAPE;
}

// out = skip + branch * row_scale without a LayerNorm behind it: the last residual connection of a Block
// (model.py:602-604) going forward, and with skip absent the gradient of its branch going back
// (dbranch = dout * row_scale), each tensor in its own dtype. 8 channels per thread; c is a multiple of 8.
__global__ __launch_bounds__(256) void scaled_add_kernel(AnyRows skip, AnyRows branch, AnyRows row_scale, int64_t n, int c,
                                                         AnyRowsOut out) {
    const int64_t groups = n * (c / 8);
    for (int64_t gi = (int64_t)blockIdx.x * 256 + threadIdx.x; gi < groups; gi += (int64_t)gridDim.x * 256) {
        const int64_t off = gi * 8;
        const Raw8 rb = raw8_load(branch.p, branch.dtype, off);
        Raw8 rs = rb;
        if (skip.p) rs = raw8_load(skip.p, skip.dtype, off);
        const float m = row_scale.p ? load1_any(row_scale.p, row_scale.dtype, off / c) : 1.f;
        float xv[8];
        raw8_floats(rb, branch.dtype, xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) xv[i] *= m;
        if (skip.p) {
            float sv[8];
            raw8_floats(rs, skip.dtype, sv);
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] += sv[i];
        }
        store8_any(out.p, out.dtype, off, xv);
    }
}

// ---- BatchNorm1d in training mode (+ exact GELU)
__device__ __forceinline__ float gelu_grad(float z) {
    const float cdf = 0.5f * (1.f + erff(z * 0.70710678118654752f));
    return cdf + z * 0.3989422804014327f * __expf(-0.5f * z * z);
}

// adds every lane's eight column values up over the rows a wave holds side by side, the waves and, with one
// atomic per channel, the work-groups: out[ch] += ..., out2[ch] += ...
template <int LPR>
__device__ __forceinline__ void column_sums_out(float* a, float* b, float (*part)[4][LPR * 8], float* out, float* out2) {
    constexpr int C = LPR * 8;
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int sub = lane % LPR, rsub = lane / LPR;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int off = LPR; off < PTV3_WAVE; off <<= 1) {
            a[i] += __shfl_xor(a[i], off, PTV3_WAVE);
            b[i] += __shfl_xor(b[i], off, PTV3_WAVE);
        }
    }
    if (rsub == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            part[0][wave][sub * 8 + i] = a[i];
            part[1][wave][sub * 8 + i] = b[i];
        }
    }
    __syncthreads();
    for (int c = tid; c < 2 * C; c += 256) {
        const int which = c / C, ch = c % C;
        const float v = part[which][0][ch] + part[which][1][ch] + part[which][2][ch] + part[which][3][ch];
        atomicAdd((which ? out2 : out) + ch, v);
    }
}

// sums[0][ch] += sum_rows (x - x[0][ch]), sums[1][ch] += sum_rows (x - x[0][ch])^2
template <int LPR>
__global__ __launch_bounds__(256) void bn_stats_kernel(AnyRows x, int64_t n, float* __restrict__ sums) {
    constexpr int C = LPR * 8, RPW = PTV3_WAVE / LPR;
    __shared__ float part[2][4][C];
    const int wave = threadIdx.x / PTV3_WAVE, lane = threadIdx.x % PTV3_WAVE;
    const int sub = lane % LPR, rsub = lane / LPR;
    float pivot[8], s1[8], s2[8];
    load8_any(x.p, x.dtype, sub * 8, pivot);
#pragma unroll
    for (int i = 0; i < 8; ++i) { s1[i] = 0.f; s2[i] = 0.f; }
    const int64_t stride = (int64_t)gridDim.x * 4 * RPW;
    for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW; row0 < n; row0 += stride) {
        const int64_t row = row0 + rsub;
        if (row < n) {
            float v[8];
            raw8_floats(raw8_load(x.p, x.dtype, row * C + sub * 8), x.dtype, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float d = v[i] - pivot[i];
                s1[i] += d;
                s2[i] = fmaf(d, d, s2[i]);
            }
        }
    }
    column_sums_out<LPR>(s1, s2, part, sums, sums + C);
}

// one work-group: stats[0] = mean, stats[1] = rstd from the sums above; running averages updated in place
// (unbiased variance, as torch does), when given
__global__ __launch_bounds__(256) void bn_finalize_kernel(AnyRows x, const float* __restrict__ sums, int64_t n, int c,
                                                          float eps, float momentum, float* __restrict__ running_mean,
                                                          float* __restrict__ running_var, float* __restrict__ stats) {
    for (int ch = threadIdx.x; ch < c; ch += 256) {
        const float pivot = load1_any(x.p, x.dtype, ch);
        const float m1 = sums[ch] / (float)n;
        const float var = fmaxf(sums[c + ch] / (float)n - m1 * m1, 0.f);
        const float mean = pivot + m1;
        stats[ch] = mean;
        stats[c + ch] = rsqrtf(var + eps);
        stats[2 * c + ch] = var;
        if (running_mean) {
            running_mean[ch] = (1.f - momentum) * running_mean[ch] + momentum * mean;
            const float unbiased = n > 1 ? var * ((float)n / (float)(n - 1)) : var;
            running_var[ch] = (1.f - momentum) * running_var[ch] + momentum * unbiased;
        }
    }
}

// PASS 0: sums[0][ch] += sum_rows dz * xhat, sums[1][ch] += sum_rows dz.
// PASS 1: dx = gamma * rstd * (dz - sums[1] / n - xhat * sums[0] / n), or gamma * rstd * dz when the statistics
// were not the batch's own (evaluation mode). dz = dy * gelu'(gamma * xhat + beta) with GELU, else dy.
template <int LPR, int PASS>
__global__ __launch_bounds__(256) void bn_bwd_kernel(AnyRows x, AnyRows dy, const float* __restrict__ stats,
                                                     AnyRows gamma, AnyRows beta, int64_t n, int gelu, int batch_stats,
                                                     float* __restrict__ sums, AnyRowsOut dx) {
    constexpr int C = LPR * 8, RPW = PTV3_WAVE / LPR;
    __shared__ float part[2][4][C];
    const int wave = threadIdx.x / PTV3_WAVE, lane = threadIdx.x % PTV3_WAVE;
    const int sub = lane % LPR, rsub = lane / LPR;
    float mean[8], rstd[8], g[8], b[8], a1[8], a2[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        mean[i] = stats[sub * 8 + i];
        rstd[i] = stats[C + sub * 8 + i];
        g[i] = 1.f;
        b[i] = 0.f;
        a1[i] = 0.f;
        a2[i] = 0.f;
    }
    if (gamma.p) load8_any(gamma.p, gamma.dtype, sub * 8, g);
    if (beta.p) load8_any(beta.p, beta.dtype, sub * 8, b);
    if (PASS == 1) {
        const float inv_n = batch_stats ? 1.f / (float)n : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a1[i] = sums[sub * 8 + i] * inv_n;       // mean of dz * xhat
            a2[i] = sums[C + sub * 8 + i] * inv_n;   // mean of dz
        }
    }
    const int64_t stride = (int64_t)gridDim.x * 4 * RPW;
    for (int64_t row0 = ((int64_t)blockIdx.x * 4 + wave) * RPW; row0 < n; row0 += stride) {
        const int64_t row = row0 + rsub;
        if (row < n) {
            const int64_t off = row * C + sub * 8;
            const Raw8 rx = raw8_load(x.p, x.dtype, off);
            const Raw8 rg = raw8_load(dy.p, dy.dtype, off);
            float xv[8], dz[8];
            raw8_floats(rx, x.dtype, xv);
            raw8_floats(rg, dy.dtype, dz);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                xv[i] = (xv[i] - mean[i]) * rstd[i];   // xhat
                if (gelu) dz[i] *= gelu_grad(fmaf(g[i], xv[i], b[i]));
            }
            if (PASS == 0) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a1[i] = fmaf(dz[i], xv[i], a1[i]);
                    a2[i] += dz[i];
                }
            } else {
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = g[i] * rstd[i] * (dz[i] - a2[i] - xv[i] * a1[i]);
                store8_any(dx.p, dx.dtype, off, o);
            }
        }
    }
    if (PASS == 0) column_sums_out<LPR>(a1, a2, part, sums, sums + C);
}

template <int PASS>
int launch_bn_bwd(AnyRows x, AnyRows dy, const float* stats, AnyRows gamma, AnyRows beta, int64_t n, int c, int gelu,
                  int batch_stats, float* sums, AnyRowsOut dx, hipStream_t stream) {
#define PTV3_BNB(L)                                                                                                   \
    if (c == 8 * L) {                                                                                                 \
        hipLaunchKernelGGL((bn_bwd_kernel<L, PASS>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0, stream, x, dy,      \
                           stats, gamma, beta, n, gelu, batch_stats, sums, dx);                                       \
        PTV3_RETURN_LAUNCH();                                                                                         \
    }
    PTV3_BNB(4) PTV3_BNB(8) PTV3_BNB(16) PTV3_BNB(32) PTV3_BNB(64)
#undef PTV3_BNB
    return PTV3_ESHAPE;
}

bool ln_dtype_ok(int dtype) { return dtype >= PTV3_F32 && dtype <= PTV3_BF16; }
bool ln_channels_ok(int c) { return c == 32 || c == 64 || c == 128 || c == 256 || c == 512; }

// The output voxel of every pair of a tap-major pair list: pair q's product row has slot pair_slot[q], and the
// slots of voxel i are [row_ptr[i], row_ptr[i + 1]).
__global__ __launch_bounds__(256) void pair_out_kernel(const int32_t* __restrict__ row_ptr,
                                                       const int32_t* __restrict__ pair_slot, int64_t n, int64_t n_pairs,
                                                       int32_t* __restrict__ pair_out) {
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= n_pairs) return;
    const int32_t slot = pair_slot[q];
    int64_t lo = 0, hi = n - 1;   // the last voxel whose first slot is at or before this one
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (row_ptr[mid] <= slot) lo = mid;
        else hi = mid - 1;
    }
    pair_out[q] = (int32_t)lo;
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

int outer_cu_count() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 1)
            v = 256;
        cus = v;
    }
    return cus;
}

// Rows of the reduction per work-group. Two work-groups fit a CU, and they all start together: the launch takes
// as long as the CU with the most of them, so a count just above a multiple of 2 x CUs costs a whole round more
// (measured: 516 work-groups 55 us, 444 of the same layer 45 us). The number of ranges minimises
// rounds x (rows per range + what a work-group costs apart from its rows: its block of the result written and
// read again by the sum over ranges, about 384 rows' worth), rounds counted on the XCD that gets the most
// (tap, range) pairs (see outer_item). The gathering form keeps its pair list in LDS (cap rows per range) and
// runs several rounds anyway: about 1024 work-groups of at least 1024 rows.
void outer_split(int64_t n, int64_t blocks, int taps, int64_t cap, int64_t* splits, int64_t* rows) {
    const int64_t slots_per_xcd = 2 * outer_cu_count() / XCDS, fixed = 384;
    int64_t best = ptv3_ceil_div(1024, blocks * taps);
    if (best > ptv3_ceil_div(n, 1024)) best = ptv3_ceil_div(n, 1024);
    if (best < 1) best = 1;
    if (cap <= 0) {
        int64_t hi = 4 * slots_per_xcd * XCDS / (blocks * taps);
        const int64_t most = ptv3_ceil_div(n, 256);
        if (hi > most) hi = most;
        int64_t best_cost = INT64_MAX;
        for (int64_t s = 1; s <= hi; ++s) {
            const int64_t on_xcd = ptv3_ceil_div(taps * s, XCDS) * blocks;
            const int64_t cost = ptv3_ceil_div(on_xcd, slots_per_xcd) * (ptv3_ceil_div(n, s) + fixed);
            if (cost < best_cost) { best_cost = cost; best = s; }
        }
    }
    int64_t r = ptv3_ceil_div(ptv3_ceil_div(n, best), 128) * 128;
    if (cap > 0 && r > cap) r = cap;
    *rows = r;
    *splits = ptv3_ceil_div(n, r);
}

// block side: 128 when both sides of the result have that many channels, else 64
int outer_side(int m_total, int k_total) { return (m_total >= OW_C && k_total >= OW_C) ? OW_C : OR_C; }

template <bool GATHER>
size_t outer_workspace(int64_t n, int m_total, int k_total, int taps) {
    const int side = outer_side(m_total, k_total);
    int64_t splits, rows;
    outer_split(n, ptv3_ceil_div(m_total, side) * ptv3_ceil_div(k_total, side), taps, GATHER ? OR_LIST : 0, &splits, &rows);
    return splits > 1 ? ptv3_align256((size_t)splits * ((size_t)m_total * taps * k_total + m_total) * sizeof(float)) : 0;
}

// d (m_total, taps, k_total) fp32 is written in full; so is colsum (m_total,) when given: the column sums of a
template <typename T, bool GATHER>
int launch_outer(const void* a, const void* b, int64_t n, int m_total, int k_total, const int32_t* nbr, int taps,
                 float* d, float* colsum, void* workspace, size_t workspace_bytes, hipStream_t stream,
                 const int32_t* tap_ptr = nullptr, const int32_t* pair_in = nullptr) {
    const int side = outer_side(m_total, k_total);
    const int64_t bm = ptv3_ceil_div(m_total, side), bk = ptv3_ceil_div(k_total, side);
    int64_t splits, rows;
    outer_split(n, bm * bk, taps, GATHER ? OR_LIST : 0, &splits, &rows);
    if ((int64_t)taps * splits >= (1ll << 31)) return PTV3_EINVAL;
    const int64_t count = (int64_t)m_total * taps * k_total;
    const int64_t stride = count + m_total;
    if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * stride * sizeof(float))) return PTV3_EWORKSPACE;
    float* slabs = splits > 1 ? (float*)workspace : d;
    float* cols = !colsum ? nullptr : (splits > 1 ? slabs + count : colsum);
    const int64_t items = ptv3_ceil_div((int64_t)taps * splits, XCDS) * XCDS * bm * bk;   // see outer_item
    if (items >= (1ll << 31)) return PTV3_EINVAL;
    const dim3 grid((unsigned)items);
    if (side == OW_C)
        hipLaunchKernelGGL((outer_rows_wide_kernel<T, GATHER>), grid, dim3(256), 0, stream, (const T*)a, (const T*)b, n,
                           m_total, k_total, nbr, tap_ptr, pair_in, taps, (int)splits, rows, stride, slabs, cols);
    else
        hipLaunchKernelGGL((outer_rows_kernel<T, GATHER>), grid, dim3(256), 0, stream, (const T*)a, (const T*)b, n,
                           m_total, k_total, nbr, tap_ptr, pair_in, taps, (int)splits, rows, stride, slabs, cols);
    if (splits > 1) {
        if (tap_ptr && count >= (1ll << 31)) return PTV3_EINVAL;
        const int64_t total = colsum ? stride : count;
        hipLaunchKernelGGL(slab_sum_kernel, dim3((unsigned)ptv3_ceil_div(total, 32)), dim3(256), 0, stream,
                           (const float*)slabs, stride, total, (int)splits, d, count, colsum, tap_ptr, taps, k_total, rows);
    }
    PTV3_RETURN_LAUNCH();
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
    const int64_t count = (int64_t)cout * taps * cin;
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(count, 256)), dim3(256), 0, stream, dw, count);
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

static bool wgrad_on_mfma(int dtype, int cin, int cout) {
    return dtype != PTV3_F32 && cin % 8 == 0 && cout % 8 == 0;
}

extern "C" size_t ptv3_subm_conv_wgrad_workspace_bytes(int dtype, int64_t n, int cin, int cout, int taps) {
    if (n < 1 || cin < 1 || cout < 1 || taps < 1 || !wgrad_on_mfma(dtype, cin, cout)) return 0;
    return outer_workspace<true>(n, cout, cin, taps);
}

extern "C" int ptv3_subm_conv_wgrad(const void* feat, const void* dout, int dtype, int64_t n, int cin, int cout,
                                    const int32_t* nbr, int taps, float* dweight, float* dbias, void* workspace,
                                    size_t workspace_bytes, void* stream_) {
    if (n < 0 || cin < 1 || cout < 1 || taps < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (!dweight) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dbias && !wgrad_on_mfma(dtype, cin, cout)) return PTV3_ESHAPE;   // the bias sum rides on the matrix-core kernel only
    if (n == 0) {
        const int64_t count = (int64_t)cout * taps * cin;
        hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(count, 256)), dim3(256), 0, stream, dweight, count);
        if (dbias) hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(cout, 256)), dim3(256), 0, stream, dbias, (int64_t)cout);
        PTV3_RETURN_LAUNCH();
    }
    if (!feat || !dout || !nbr) return PTV3_EINVAL;
    if ((int64_t)taps * ptv3_ceil_div(n, 256) >= (1ll << 31)) return PTV3_EINVAL;
    if (wgrad_on_mfma(dtype, cin, cout)) {
        if (dtype == PTV3_F16)
            return launch_outer<_Float16, true>(dout, feat, n, cout, cin, nbr, taps, dweight, dbias, workspace, workspace_bytes, stream);
        return launch_outer<__bf16, true>(dout, feat, n, cout, cin, nbr, taps, dweight, dbias, workspace, workspace_bytes, stream);
    }
    if (dtype == PTV3_F16) return launch_wgrad<_Float16>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
    if (dtype == PTV3_BF16) return launch_wgrad<__bf16>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
    return launch_wgrad<float>(feat, dout, n, cin, cout, nbr, taps, dweight, stream);
}

extern "C" int ptv3_conv_plan_pair_out(const int32_t* row_ptr, const int32_t* pair_slot, int64_t n, int64_t n_pairs,
                                       int32_t* pair_out, void* stream_) {
    if (n < 0 || n_pairs < 0) return PTV3_EINVAL;
    if (n == 0 || n_pairs == 0) return PTV3_OK;
    if (!row_ptr || !pair_slot || !pair_out) return PTV3_EINVAL;
    hipLaunchKernelGGL(pair_out_kernel, dim3((unsigned)ptv3_ceil_div(n_pairs, 256)), dim3(256), 0, (hipStream_t)stream_,
                       row_ptr, pair_slot, n, n_pairs, pair_out);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_subm_conv_wgrad_pairs(const void* feat, const void* dout, int dtype, int64_t n, int cin, int cout,
                                          const int32_t* tap_ptr, const int32_t* pair_in, const int32_t* pair_out,
                                          int taps, float* dweight, float* dbias, void* workspace,
                                          size_t workspace_bytes, void* stream_) {
    if (n < 1 || cin < 1 || cout < 1 || taps < 1) return PTV3_EINVAL;
    if (!wgrad_on_mfma(dtype, cin, cout)) return PTV3_ESHAPE;
    if (!feat || !dout || !tap_ptr || !pair_in || !pair_out || !dweight) return PTV3_EINVAL;
    if ((int64_t)taps * ptv3_ceil_div(n, 256) >= (1ll << 31)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16)
        return launch_outer<_Float16, true>(dout, feat, n, cout, cin, pair_out, taps, dweight, dbias, workspace,
                                            workspace_bytes, stream, tap_ptr, pair_in);
    return launch_outer<__bf16, true>(dout, feat, n, cout, cin, pair_out, taps, dweight, dbias, workspace,
                                      workspace_bytes, stream, tap_ptr, pair_in);
}

extern "C" size_t ptv3_linear_wgrad_workspace_bytes(int64_t n, int k, int nout) {
    if (n < 1 || k < 1 || nout < 1) return 0;
    return outer_workspace<false>(n, nout, k, 1);
}

extern "C" int ptv3_linear_wgrad(const void* x, const void* dout, int dtype, int64_t n, int k, int nout, float* dweight,
                                 float* dbias, void* workspace, size_t workspace_bytes, void* stream_) {
    if (n < 0 || k < 1 || nout < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (k % 8 != 0 || nout % 8 != 0) return PTV3_ESHAPE;
    if (!dweight) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (n == 0) {
        const int64_t count = (int64_t)nout * k;
        hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(count, 256)), dim3(256), 0, stream, dweight, count);
        if (dbias) hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(nout, 256)), dim3(256), 0, stream, dbias, (int64_t)nout);
        PTV3_RETURN_LAUNCH();
    }
    if (!x || !dout) return PTV3_EINVAL;
    if (dtype == PTV3_F16)
        return launch_outer<_Float16, false>(dout, x, n, nout, k, nullptr, 1, dweight, dbias, workspace, workspace_bytes, stream);
    return launch_outer<__bf16, false>(dout, x, n, nout, k, nullptr, 1, dweight, dbias, workspace, workspace_bytes, stream);
}

extern "C" int ptv3_add_layer_norm_fwd(const void* skip, int skip_dtype, const void* branch, int branch_dtype,
                                       const void* row_scale, int row_scale_dtype, const void* gamma, const void* beta,
                                       int param_dtype, int64_t n, int c, float eps, void* sum, int sum_dtype, void* y,
                                       int y_dtype, const void* pre_gamma, const void* pre_beta, float pre_eps,
                                       void* stream_) {
    if (n < 0 || c < 1) return PTV3_EINVAL;
    if (!ln_dtype_ok(skip_dtype) || !ln_dtype_ok(branch_dtype) || !ln_dtype_ok(row_scale_dtype) ||
        !ln_dtype_ok(param_dtype) || !ln_dtype_ok(sum_dtype) || !ln_dtype_ok(y_dtype))
        return PTV3_EINVAL;
    if (!ln_channels_ok(c)) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!branch || !gamma || !beta || !y || (pre_gamma == nullptr) != (pre_beta == nullptr)) return PTV3_EINVAL;
    return launch_add_ln_fwd({skip, skip_dtype}, {branch, branch_dtype}, {row_scale, row_scale_dtype},
                             {gamma, param_dtype}, {beta, param_dtype}, n, c, eps, {sum, sum_dtype}, {y, y_dtype},
                             {pre_gamma, param_dtype}, {pre_beta, param_dtype}, pre_eps, (hipStream_t)stream_);
}

extern "C" int ptv3_scaled_add(const void* skip, int skip_dtype, const void* branch, int branch_dtype,
                               const void* row_scale, int row_scale_dtype, int64_t n, int c, void* out, int out_dtype,
                               void* stream_) {
    if (n < 0 || c < 1) return PTV3_EINVAL;
    if (!ln_dtype_ok(skip_dtype) || !ln_dtype_ok(branch_dtype) || !ln_dtype_ok(row_scale_dtype) || !ln_dtype_ok(out_dtype))
        return PTV3_EINVAL;
    if (c % 8 != 0) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!branch || !out) return PTV3_EINVAL;
    const int64_t groups = n * (c / 8);
    const int64_t blocks = ptv3_ceil_div(groups, 256);
    hipLaunchKernelGGL(scaled_add_kernel, dim3((unsigned)(blocks < 8192 ? blocks : 8192)), dim3(256), 0,
                       (hipStream_t)stream_, AnyRows{skip, skip_dtype}, AnyRows{branch, branch_dtype},
                       AnyRows{row_scale, row_scale_dtype}, n, c, AnyRowsOut{out, out_dtype});
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_add_layer_norm_bwd(const void* sum, int sum_dtype, const void* dy, int dy_dtype, const void* dsum,
                                       int dsum_dtype, const void* row_scale, int row_scale_dtype, const void* gamma,
                                       int param_dtype, int64_t n, int c, float eps, void* dskip, int dskip_dtype,
                                       void* dbranch, int dbranch_dtype, float* dgamma, float* dbeta, const void* pre_x,
                                       int pre_x_dtype, const void* pre_gamma, float pre_eps, float* dpre_gamma,
                                       float* dpre_beta, void* stream_) {
    if (n < 0 || c < 1) return PTV3_EINVAL;
    if (!ln_dtype_ok(sum_dtype) || !ln_dtype_ok(dy_dtype) || !ln_dtype_ok(dsum_dtype) || !ln_dtype_ok(row_scale_dtype) ||
        !ln_dtype_ok(param_dtype) || !ln_dtype_ok(dskip_dtype) || !ln_dtype_ok(dbranch_dtype) || !ln_dtype_ok(pre_x_dtype))
        return PTV3_EINVAL;
    if (!ln_channels_ok(c)) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!sum || !dy || !gamma || !dgamma || !dbeta) return PTV3_EINVAL;
    if (pre_x && (!pre_gamma || !dpre_gamma || !dpre_beta)) return PTV3_EINVAL;
    return launch_add_ln_bwd({sum, sum_dtype}, {dy, dy_dtype}, {dsum, dsum_dtype}, {row_scale, row_scale_dtype},
                             {gamma, param_dtype}, n, c, eps, {dskip, dskip_dtype}, {dbranch, dbranch_dtype}, dgamma,
                             dbeta, {pre_x, pre_x_dtype}, {pre_gamma, param_dtype}, pre_eps, dpre_gamma, dpre_beta,
                             (hipStream_t)stream_);
}

extern "C" int ptv3_batch_norm_stats(const void* x, int dtype, int64_t n, int c, float eps, float momentum,
                                     float* running_mean, float* running_var, float* stats, float* workspace,
                                     void* stream_) {
    if (n < 1 || c < 1) return PTV3_EINVAL;
    if (!ln_dtype_ok(dtype)) return PTV3_EINVAL;
    if (!ln_channels_ok(c)) return PTV3_ESHAPE;
    if (!x || !stats || !workspace || ((running_mean == nullptr) != (running_var == nullptr))) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const AnyRows xr = {x, dtype};
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(2 * c, 256)), dim3(256), 0, stream, workspace, (int64_t)2 * c);
#define PTV3_BNS(L)                                                                                                   \
    if (c == 8 * L)                                                                                                   \
        hipLaunchKernelGGL((bn_stats_kernel<L>), dim3((unsigned)ln_grid(n, c)), dim3(256), 0, stream, xr, n, workspace);
    PTV3_BNS(4) PTV3_BNS(8) PTV3_BNS(16) PTV3_BNS(32) PTV3_BNS(64)
#undef PTV3_BNS
    hipLaunchKernelGGL(bn_finalize_kernel, dim3(1), dim3(256), 0, stream, xr, (const float*)workspace, n, c, eps, momentum,
                       running_mean, running_var, stats);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_batch_norm_bwd(const void* x, int x_dtype, const void* dout, int dout_dtype, const float* stats,
                                   const void* gamma, const void* beta, int param_dtype, int64_t n, int c, int gelu,
                                   int batch_stats, void* dx, int dx_dtype, float* dgamma_dbeta, void* stream_) {
    if (n < 0 || c < 1) return PTV3_EINVAL;
    if (!ln_dtype_ok(x_dtype) || !ln_dtype_ok(dout_dtype) || !ln_dtype_ok(param_dtype) || !ln_dtype_ok(dx_dtype))
        return PTV3_EINVAL;
    if (!ln_channels_ok(c)) return PTV3_ESHAPE;
    if (!dgamma_dbeta) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)ptv3_ceil_div(2 * c, 256)), dim3(256), 0, stream, dgamma_dbeta, (int64_t)2 * c);
    if (n == 0) PTV3_RETURN_LAUNCH();
    if (!x || !dout || !stats || !dx) return PTV3_EINVAL;
    const AnyRows xr = {x, x_dtype}, gr = {dout, dout_dtype}, ga = {gamma, param_dtype}, be = {beta, param_dtype};
    const AnyRowsOut out = {dx, dx_dtype};
    int rc = launch_bn_bwd<0>(xr, gr, stats, ga, be, n, c, gelu, batch_stats, dgamma_dbeta, out, stream);
    if (rc != PTV3_OK) return rc;
    return launch_bn_bwd<1>(xr, gr, stats, ga, be, n, c, gelu, batch_stats, dgamma_dbeta, out, stream);
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
