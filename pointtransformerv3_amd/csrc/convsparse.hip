// Submanifold 3x3x3 convolution, sparse tile form: work in proportion to the pairs, no pair matrix in memory.
//
// Replaces spconv.SubMConv3d.forward at the xCPE call sites of the reference (model.py:546-552:
// in_channels == out_channels, 3x3x3, bias) where a voxel has only a few of its 26 neighbours (the fine
// levels: 2 to 6 pairs per voxel). There the tile form in convtile.hip multiplies mostly rows of zeros
// (an MFMA column is an output voxel, present or not), and the pair form sends one product row per pair
// through memory and back.
//
// Here a work-group is ONE wave that owns 128 consecutive output voxels (a tile of the plan made by
// ptv3_conv_plan_tiles: the tile's pairs sorted by tap) and a slice of the output channels. Its sums live
// in LDS as fp32. It walks the tile's pairs tap by tap in blocks of up to 32: the block's input rows are
// gathered straight into MFMA operand order (a lane is a pair and a half of the 16-channel step: 16 bytes
// of its pair's row per step), are multiplied with the tap's weights (v_mfma_f32_32x32x16: an MFMA
// column is a real pair) on top of the LDS sums of the pairs' output voxels (read as the MFMAs' C operand,
// written back: the wave owns its sums alone, LDS atomics measured many times slower). The taps are walked
// in order, so the additions happen in a fixed order: no barrier, nothing shared, results reproducible. At the end the sums (which started at the
// bias) are rounded and written out in whole rows.
//
// Everything a block needs from memory is requested several blocks ahead into rings of registers: first
// the block's pair words, then (with the input rows known) the rows and the tap's weights. All loads are
// unconditional (blocks past the end repeat the last one, columns past a block's count repeat its last pair
// and add into a spare row of the sums), so the number of loads in flight is fixed and waiting for one
// block leaves the younger ones in flight.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct SpOps;
template <> struct SpOps<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
};
template <> struct SpOps<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
};

constexpr int SP_TV = 128;           // output voxels of a plan tile (ptv3_conv_plan_tiles)
constexpr int SP_TAPS = 27;
constexpr int SP_TILE_WORDS = 32;    // int32 per tile in tile_tap
constexpr int SP_IN_MASK = (1 << 24) - 1;
constexpr int SP_BLOCK = 32;         // pairs per block: the rows of one MFMA
constexpr int SP_MAX_ITEMS = SP_TAPS + SP_TV * SP_TAPS / SP_BLOCK;   // 135

template <int C, int CW>
struct SparseShape {
    static constexpr int KS = C / 16;                 // MFMA steps along the input channels
    static constexpr int CB = CW / 32;                // 32-wide output channel blocks of the work-group
    // blocks in flight; the hardware counts at most 63 outstanding loads
    static constexpr int LOADS = 1 + KS + CB * KS;    // per block: pair words, input rows, weights
    static constexpr int DEPTH = 48 / LOADS > 4 ? 4 : 48 / LOADS;
    static_assert(DEPTH >= 1 && DEPTH * LOADS + DEPTH <= 63, "loads in flight");
};

template <typename T, int C, int CW>
__global__ __launch_bounds__(64) void conv_sparse_kernel(const T* __restrict__ feat, int64_t n,
                                                         const T* __restrict__ packed_w, const T* __restrict__ bias,
                                                         const int32_t* __restrict__ tile_tap,
                                                         const uint32_t* __restrict__ tile_pair, T* __restrict__ out) {
    typedef SparseShape<C, CW> S;
    typedef typename SpOps<T>::v8 v8;
    constexpr int KS = S::KS, CB = S::CB, D = S::DEPTH;
    constexpr int SS = CW + 4;   // floats per row of sums: 4 of padding spread the rows over the banks
    __shared__ __align__(16) float sums[(SP_TV + 1) * SS];   // row SP_TV: where columns past a block's count add
    __shared__ uint32_t items[SP_MAX_ITEMS + 1];

    const int lane = threadIdx.x, col = lane & 31, hf = lane >> 5;
    // work-group ids go round the XCDs: every XCD works through one contiguous eighth of the tiles, so that tiles
    // which gather the same neighbour rows (voxels of a pooled level are in curve order) meet in one L2
    const int tile = xcd_chunked_id(blockIdx.x, gridDim.x);
    const int cout0 = blockIdx.y * CW;
    const int64_t v0 = (int64_t)tile * SP_TV;
    const int nv = (int)min((int64_t)SP_TV, n - v0);

    // ---- the tile's blocks: tap | first pair (relative to the tile's) << 5 | pairs << 20
    const int32_t* tt = tile_tap + (int64_t)tile * SP_TILE_WORDS;
    const uint32_t* tp = tile_pair + tt[28];
    int n_items;
    {
        const int first = lane < 28 ? tt[lane] : 0;
        const int next = __shfl_down(first, 1, PTV3_WAVE);
        const int c = lane < SP_TAPS ? next - first : 0;
        const int nb = (c + SP_BLOCK - 1) / SP_BLOCK;
        int x = nb;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) {
            const int y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        for (int j = 0; j < nb; ++j)
            items[x - nb + j] = (uint32_t)lane | (uint32_t)(first + j * SP_BLOCK) << 5 |
                                (uint32_t)min(SP_BLOCK, c - j * SP_BLOCK) << 20;
        n_items = __builtin_amdgcn_readlane(x, SP_TAPS - 1);   // >= 1: every voxel pairs with itself
    }
    // ---- sums start at the bias
    {
        constexpr int Q = CW / 4;   // float4 per row; 64 % Q == 0: a lane keeps its columns
        f32x4 b4 = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
#pragma unroll
            for (int j = 0; j < 4; ++j) b4[j] = (float)bias[cout0 + (lane % Q) * 4 + j];
        }
#pragma unroll 4
        for (int e = lane; e < SP_TV * Q; e += 64) *(f32x4*)(sums + (e / Q) * SS + (e % Q) * 4) = b4;
    }
    __builtin_amdgcn_wave_barrier();   // the block table is read next (LDS serves a wave's accesses in order)
    if (n_items == 0) {   // no pairs at all (never for a submanifold map, whose voxels pair with themselves): bias rows
        constexpr int E0 = CW / 8;
        for (int e = lane; e < nv * E0; e += 64) {
            const int r = e / E0, c8 = e % E0;
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o[j] = SpOps<T>::pack2(bias ? (float)bias[cout0 + c8 * 8 + 2 * j] : 0.f,
                                       bias ? (float)bias[cout0 + c8 * 8 + 2 * j + 1] : 0.f);
            *(u32x4*)(out + (v0 + r) * C + cout0 + c8 * 8) = o;
        }
        return;
    }

    // descriptors of the blocks k0 .. k0 + 2D - 1 (da) and k0 + 2D .. k0 + 4D - 1 (db) as scalars: one LDS read per
    // 2D blocks; past the end the last block repeats (its loads are valid, its products go to the spare row)
    const int last = n_items - 1;
    auto fetch = [&](int k0, uint32_t (&dst)[2 * S::DEPTH]) {
        const uint32_t mine = items[min(k0 + (lane & 15), last)];
#pragma unroll
        for (int j = 0; j < 2 * S::DEPTH; ++j) dst[j] = (uint32_t)__builtin_amdgcn_readlane((int)mine, j);
    };
    uint32_t da[2 * S::DEPTH], db[2 * S::DEPTH];
    fetch(0, da);
    fetch(2 * S::DEPTH, db);
    const T* wbase = packed_w + ((int64_t)(cout0 / 32) * KS * 64 + lane) * 8;
    constexpr int64_t W_TAP = (int64_t)(C / 32) * KS * 64 * 8;   // halfs per tap

    // words[k % 2D]: the pair words of block k (lane's pair: lane % 32), requested 2 D blocks ahead; x / w[k % D]: the
    // pairs' input rows, already in MFMA operand order (lane (pair, half) takes channels 16 i + 8 half .. + 8 of its
    // pair's row), and the tap's weights, requested D blocks ahead
    uint32_t words[2 * D];
    u32x4 x[D][KS], w[D][CB * KS];
    auto load_words = [&](uint32_t d) -> uint32_t {
        const int start = (int)((d >> 5) & 0x7fff), cnt = (int)(d >> 20);
        return tp[start + min(col, cnt - 1)];
    };
    auto issue = [&](uint32_t d, uint32_t kw, int s) {
        const int t = (int)(d & 31);
        const T* row = feat + (int64_t)(kw & SP_IN_MASK) * C + hf * 8;
#pragma unroll
        for (int i = 0; i < KS; ++i) x[s][i] = *(const u32x4*)(row + i * 16);
#pragma unroll
        for (int i = 0; i < CB * KS; ++i) w[s][i] = *(const u32x4*)(wbase + t * W_TAP + (int64_t)i * 64 * 8);
    };
    auto compute = [&](int cnt, uint32_t kw, int s) {
        // an MFMA column is a pair: this lane's 16 products are output channels 8 (v / 4) + 4 hf + v % 4 of the
        // output voxel of pair `col`, whose word this lane holds
        // The columns are different pairs of one tap, so different output voxels (or the spare row): the sums so
        // far enter the products as the MFMAs' C operand, and what comes out is written back.
        float* mine = sums + (col < cnt ? (int)(kw >> 24) : SP_TV) * SS + 4 * hf;
        f32x16 acc[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 old = *(const f32x4*)(mine + cb * 32 + 8 * q);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[cb][4 * q + j] = old[j];
            }
        }
#pragma unroll
        for (int i = 0; i < KS; ++i) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                acc[cb] = SpOps<T>::mfma(__builtin_bit_cast(v8, w[s][cb * KS + i]), __builtin_bit_cast(v8, x[s][i]), acc[cb]);
        }
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4 nw;
#pragma unroll
                for (int j = 0; j < 4; ++j) nw[j] = acc[cb][4 * q + j];
                *(f32x4*)(mine + cb * 32 + 8 * q) = nw;
            }
        }
    };

    // ---- prologue: pair words of the first 2 D blocks, rows and weights of the first D
#pragma unroll
    for (int j = 0; j < 2 * D; ++j) words[j] = load_words(da[j]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < D; ++j) {
        issue(da[j], words[j], j);
        __builtin_amdgcn_sched_barrier(0);   // block 0's loads first: the loop waits for them first
    }
    for (int k0 = 0; k0 < n_items; k0 += 2 * D) {
#pragma unroll
        for (int j = 0; j < 2 * D; ++j) {
            // no branch around a block: past the end its count is 0 and every column adds into the spare row
            compute(k0 + j < n_items ? (int)(da[j] >> 20) : 0, words[j], j % D);
            words[j] = load_words(db[j]);
            issue(j < D ? da[j + D] : db[j - D], words[(j + D) % (2 * D)], j % D);
            __builtin_amdgcn_sched_barrier(0);   // keep the loads in block order: the waits count them in issue order
        }
#pragma unroll
        for (int j = 0; j < 2 * D; ++j) da[j] = db[j];
        fetch(k0 + 4 * D, db);
    }

    // ---- sums -> halfs -> out, 16 bytes per lane
    constexpr int E = CW / 8;   // lanes per output row
    for (int e = lane; e < nv * E; e += 64) {
        const int r = e / E, c8 = e % E;
        const f32x4 lo = *(const f32x4*)(sums + r * SS + c8 * 8);
        const f32x4 hi = *(const f32x4*)(sums + r * SS + c8 * 8 + 4);
        u32x4 o;
        o[0] = SpOps<T>::pack2(lo[0], lo[1]);
        o[1] = SpOps<T>::pack2(lo[2], lo[3]);
        o[2] = SpOps<T>::pack2(hi[0], hi[1]);
        o[3] = SpOps<T>::pack2(hi[2], hi[3]);
        *(u32x4*)(out + (v0 + r) * C + cout0 + c8 * 8) = o;
    }
}

template <typename T, int C, int CW>
int launch_sparse(const void* feat, int64_t n, const void* packed_w, const void* bias, const int32_t* tile_tap,
                  const uint32_t* tile_pair, void* out, hipStream_t stream) {
    const dim3 grid((unsigned)ptv3_ceil_div(n, SP_TV), (unsigned)(C / CW));
    hipLaunchKernelGGL((conv_sparse_kernel<T, C, CW>), grid, dim3(64), 0, stream, (const T*)feat, n, (const T*)packed_w,
                       (const T*)bias, tile_tap, tile_pair, (T*)out);
    PTV3_RETURN_LAUNCH();
}

template <typename T>
int dispatch_sparse(const void* feat, int64_t n, int c, const void* packed_w, const void* bias, const int32_t* tile_tap,
                    const uint32_t* tile_pair, void* out, hipStream_t stream) {
    switch (c) {
        case 32: return launch_sparse<T, 32, 32>(feat, n, packed_w, bias, tile_tap, tile_pair, out, stream);
        case 64: return launch_sparse<T, 64, 64>(feat, n, packed_w, bias, tile_tap, tile_pair, out, stream);
    }
    return PTV3_ESHAPE;
}

}  // namespace

extern "C" int ptv3_subm_conv_sparse_fwd(const void* feat, int dtype, int64_t n, int channels, int taps,
                                         const void* packed_weight, const void* bias, const int32_t* tile_tap,
                                         const int32_t* tile_pair, void* out, void* stream_) {
    if (n < 0 || n >= (1ll << 24)) return PTV3_EINVAL;
    if (taps != SP_TAPS) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (channels != 32 && channels != 64) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!feat || !packed_weight || !tile_tap || !tile_pair || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const uint32_t* tp = (const uint32_t*)tile_pair;
    if (dtype == PTV3_F16) return dispatch_sparse<_Float16>(feat, n, channels, packed_weight, bias, tile_tap, tp, out, stream);
    return dispatch_sparse<__bf16>(feat, n, channels, packed_weight, bias, tile_tap, tp, out, stream);
}
