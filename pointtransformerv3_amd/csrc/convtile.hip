// Submanifold 3x3x3 convolution, tile form: no pair matrix in memory.
//
// Replaces spconv.SubMConv3d.forward at the xCPE call sites of the reference (model.py:546-552:
// in_channels == out_channels, 3x3x3, bias) where the pair form's round trip of one product row
// per (input, output) pair through HBM is what bounds it (up to 256 channels).
//
// A work-group owns TV consecutive output voxels and keeps their sums as fp32 in LDS. It reads
// the voxels' pairs from the output-major list (slot_pair: tap << 24 | input row, voxel i's pairs
// at [row_ptr[i], row_ptr[i+1])), sorts them by tap in LDS (counting sort), and walks the taps in
// order: the input rows of up to 64 pairs of one tap are gathered into LDS in whole row segments,
// every wave multiplies them with its own 32 output channels of that tap's weights
// (v_mfma_f32_32x32x16, product transposed: a column is a pair), and adds its 32x32 block into the
// LDS sums of the pairs' output voxels. MFMA columns are real pairs whatever the sparsity, an
// output is written once, nothing is atomic, and the order of the additions (tap order, fp32) is
// fixed. Waves own disjoint channel slices, or disjoint pairs of the same tap, and a barrier per
// chunk orders the taps, so the read-modify-write of the sums needs no atomics.
//
// The weights come in fragment order (ptv3_subm_conv_pack_weight): the 16 bytes lane l needs for
// (tap, 32-channel slice, 16-channel step) are stored at consecutive addresses over the lanes, so a
// wave fetches a fragment as one contiguous KB straight into registers, one tap ahead; the input
// rows of the next chunk are in flight while this one is multiplied.
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

template <typename T> struct TileOps;
template <> struct TileOps<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
};
template <> struct TileOps<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
};

constexpr int CT_THREADS = 256;
constexpr int CT_TAPS = 27;
constexpr int CT_IN_MASK = (1 << 24) - 1;

// weight (c, taps, c) -> fragment order: piece ((t * c/32 + slice) * c/16 + step) * 64 + lane holds
// input channels 16 step + 8 (lane / 32) .. + 8 of output channel 32 slice + lane % 32 at tap t
template <typename T>
__global__ __launch_bounds__(CT_THREADS) void pack_weight_kernel(const T* __restrict__ w, int c, int taps,
                                                                 T* __restrict__ packed) {
    const int64_t total = (int64_t)taps * c * c / 8;
    const int64_t idx = (int64_t)blockIdx.x * CT_THREADS + threadIdx.x;
    if (idx >= total) return;
    const int lane = (int)(idx % 64);
    int64_t r = idx / 64;
    const int steps = c / 16, slices = c / 32;
    const int s = (int)(r % steps);
    r /= steps;
    const int sl = (int)(r % slices);
    const int t = (int)(r / slices);
    const int co = 32 * sl + lane % 32, k = 16 * s + 8 * (lane / 32);
    *(u32x4*)(packed + idx * 8) = *(const u32x4*)(w + ((int64_t)co * taps + t) * c + k);
}

// the same for several weights in one launch: job j owns blocks first_block[j] .. first_block[j + 1]
__global__ __launch_bounds__(CT_THREADS) void pack_weight_batch_kernel(const ptv3_pack_job* __restrict__ jobs, int n_jobs) {
    int j = 0;
    for (int i = 1; i < n_jobs; ++i)
        if (jobs[i].first_block <= (int64_t)blockIdx.x) j = i;   // uniform: a handful of jobs, first_block ascending
    const ptv3_pack_job job = jobs[j];
    const int c = job.channels, taps = job.taps;
    if (c < 32 || c % 32 != 0 || taps < 1) return;   // a row no *_blocks() helper would have sized: touch nothing
    const int64_t total = (int64_t)taps * c * c / 8;
    const int64_t idx = ((int64_t)blockIdx.x - job.first_block) * CT_THREADS + threadIdx.x;
    if (idx < 0 || idx >= total) return;
    const int lane = (int)(idx % 64);
    int64_t r = idx / 64;
    const int steps = c / 16, slices = c / 32;
    const int st = (int)(r % steps);
    r /= steps;
    const int sl = (int)(r % slices);
    const int t = (int)(r / slices);
    const int co = 32 * sl + lane % 32, k = 16 * st + 8 * (lane / 32);
    const uint16_t* w = (const uint16_t*)job.weight;   // both half types are 16-bit patterns here
    *(u32x4*)((uint16_t*)job.packed + idx * 8) = *(const u32x4*)(w + ((int64_t)co * taps + t) * c + k);
}

// output-major pair words from the tap-major lists: slot_pair[pair_slot[q]] = tap(q) << 24 | pair_in[q]
__global__ __launch_bounds__(CT_THREADS) void plan_slots_kernel(const int32_t* __restrict__ tap_ptr, int taps,
                                                                const int32_t* __restrict__ pair_in,
                                                                const int32_t* __restrict__ pair_slot, int64_t n_pairs,
                                                                int32_t* __restrict__ slot_pair) {
    __shared__ int32_t tp[129];
    for (int i = threadIdx.x; i <= taps; i += CT_THREADS) tp[i] = tap_ptr[i];
    __syncthreads();
    const int64_t q = (int64_t)blockIdx.x * CT_THREADS + threadIdx.x;
    if (q >= n_pairs) return;
    int lo = 0, hi = taps;   // largest t with tp[t] <= q: the (non-empty) tap that holds q
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tp[mid] <= (int32_t)q) lo = mid; else hi = mid;
    }
    slot_pair[pair_slot[q]] = (int32_t)((uint32_t)lo << 24 | (uint32_t)pair_in[q]);
}

constexpr int CT_TV = 128;          // output voxels per tile (the 128-channel tile form also takes tiles of 96)
constexpr int CT_TILE_WORDS = 32;   // int32 per tile in tile_tap: 28 tap starts (relative), the tile's first pair

// Per tile of blockDim.x (96 or 128) consecutive voxels: its pairs sorted by tap, inside a tap by output voxel.
// tile_tap[tile][t] = first pair of tap t relative to the tile's first pair (t = 27: the tile's pair
// count), [28] = the tile's first pair; tile_pair[.] = voxel inside the tile << 24 | input row, in that
// order; vox_taps[i] = bit t set when voxel i has a neighbour at tap t.
__global__ __launch_bounds__(CT_TV) void plan_tiles_kernel(const int32_t* __restrict__ row_ptr,
                                                           const int32_t* __restrict__ slot_pair, int64_t n,
                                                           int32_t* __restrict__ tile_tap, uint32_t* __restrict__ tile_pair,
                                                           uint32_t* __restrict__ vox_taps) {
    __shared__ int32_t wave_cnt[2][32], tstart[32];
    const int tid = threadIdx.x, lane = tid % PTV3_WAVE, wave = tid / PTV3_WAVE;
    const int64_t v0 = (int64_t)blockIdx.x * blockDim.x;
    const bool live = v0 + tid < n;
    int s_lo = 0, s_hi = 0;
    if (live) {
        s_lo = row_ptr[v0 + tid];
        s_hi = row_ptr[v0 + tid + 1];
    }
    const int32_t base = row_ptr[v0];
    uint32_t mine = 0;
    for (int s = s_lo; s < s_hi; ++s) mine |= 1u << (((uint32_t)slot_pair[s] >> 24) & 31);
    if (live) vox_taps[v0 + tid] = mine;
    for (int t = 0; t < CT_TAPS; ++t) {
        const uint64_t bal = __ballot((mine >> t) & 1u);
        if (lane == 0) wave_cnt[wave][t] = __popcll(bal);
    }
    __syncthreads();
    if (wave == 0) {
        const int c = lane < CT_TAPS ? wave_cnt[0][lane] + wave_cnt[1][lane] : 0;
        int x = c;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) {
            const int y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        if (lane < 32) {
            tstart[lane] = x - c;
            int32_t word = x - c;           // lanes 27.. hold the total
            if (lane == 28) word = base;
            tile_tap[(int64_t)blockIdx.x * CT_TILE_WORDS + lane] = word;
        }
    }
    __syncthreads();
    const uint64_t below = (1ull << lane) - 1ull;
    int s = s_lo;   // a voxel's slots follow tap order
    for (int t = 0; t < CT_TAPS; ++t) {
        const bool has = (mine >> t) & 1u;
        const uint64_t bal = __ballot(has);
        if (has) {
            const int pos = tstart[t] + (wave == 1 ? wave_cnt[0][t] : 0) + __popcll(bal & below);
            tile_pair[base + pos] = (uint32_t)tid << 24 | ((uint32_t)slot_pair[s] & CT_IN_MASK);
            ++s;
        }
    }
}

// TV_ output voxels per tile: 128, or 96 where the four waves split the output channels (128 channels): a launch
// whose 128-voxel tiles fill 2.2 rounds of the resident work-groups costs three, with 96-voxel tiles 2.97 rounds of
// tiles that are a quarter cheaper
template <int C, int TV_ = CT_TV>
struct TileShape {
    static constexpr int TV = TV_;
    static constexpr int THREADS = 256;
    static constexpr int COUT_WG = C > 128 ? 128 : C;     // output channels of a work-group
    static constexpr int CW = COUT_WG / 32;               // waves across channels
    static constexpr int PW = 4 / CW;                     // waves across the 32-voxel groups of the tile
    static constexpr int GPW = TV / 32 / PW;              // groups per wave
    static constexpr int CH = C >= 128 ? TV : 64;         // pairs per chunk (128 channels: a tap of a tile is one chunk)
    static constexpr int KS = C / 16;                     // MFMA steps along the input channels
    static constexpr int LPR = C / 8;                     // lanes (16 B each) per input row
    static constexpr int RPP = THREADS / LPR;             // rows per gather instruction of the work-group
    static constexpr int NL = CH / RPP;                   // gather instructions per chunk
    static constexpr int CAP = TV * CT_TAPS;              // pairs of a tile at most
    static constexpr int MAX_CHUNKS = CT_TAPS + CAP / CH;
    static constexpr int OCC = 2;                         // work-groups per CU the registers allow
    static constexpr int DEPTH = 2;                       // chunks in flight
    static constexpr size_t XBUF = (size_t)TV * C * 2;    // bytes of one buffer of input rows (swizzled, no padding)
    static constexpr size_t LDS = 2 * XBUF + (size_t)CAP * 4 + (size_t)C * 2;   // + one row of zeros
    static_assert(CH % RPP == 0 && NL >= 1 && MAX_CHUNKS <= 128 && LPR >= 8 && GPW * PW * 32 == TV, "tile shape");
};

// Input rows sit in LDS at the row of their OUTPUT voxel, 16-byte pieces swizzled by the row so that the
// 32 rows a fragment read touches spread over the banks without padding.
template <int C>
__device__ __forceinline__ int swz(int row, int piece) {
    return row * C + ((piece ^ (row & 7)) * 8);   // in halfs
}

template <typename T, int C, int TV_>
__global__ __launch_bounds__((TileShape<C, TV_>::THREADS), (TileShape<C, TV_>::OCC)) void conv_tile_kernel(
    const T* __restrict__ feat, int64_t n, const T* __restrict__ packed_w, const T* __restrict__ bias,
    const int32_t* __restrict__ tile_tap, const uint32_t* __restrict__ tile_pair, const uint32_t* __restrict__ vox_taps,
    T* __restrict__ out) {
    typedef TileShape<C, TV_> S;
    typedef typename TileOps<T>::v8 v8;
    constexpr int TV = S::TV, CW = S::CW, GPW = S::GPW, CH = S::CH, KS = S::KS;
    constexpr int LPR = S::LPR, RPP = S::RPP, NL = S::NL, COUT_WG = S::COUT_WG, DEPTH = S::DEPTH;
    constexpr int THREADS = S::THREADS;
    extern __shared__ __align__(16) char smem[];
    T* xs = (T*)smem;                                        // [2][TV][C] input rows by output voxel
    uint32_t* plist = (uint32_t*)(smem + 2 * S::XBUF);       // [CAP] the tile's pairs by tap
    T* zero_row = (T*)(plist + S::CAP);                      // [C] what an output without the tap multiplies
    __shared__ int32_t ch_tap[128], ch_base[128], ch_cnt[128];
    __shared__ int32_t n_chunks;

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int cw = wave % CW, pw = wave / CW;
    const int cout0 = blockIdx.y * COUT_WG;             // first output channel of the work-group
    // work-group ids go round the XCDs: every XCD works through one contiguous eighth of the tiles, so that tiles
    // which gather the same neighbour rows meet in one L2 (no faster, but half the HBM reads)
    const int tile = xcd_chunked_id(blockIdx.x, gridDim.x);
    const int64_t v0 = (int64_t)tile * TV;
    const int nv = (int)min((int64_t)TV, n - v0);

    // ---- the tile's pair list and chunk table
    const int32_t* tt = tile_tap + (int64_t)tile * CT_TILE_WORDS;
    const int total = tt[CT_TAPS];
    const uint32_t* tp = tile_pair + tt[28];
    for (int e = tid; e < total; e += THREADS) plist[e] = tp[e];
    if (tid < C / 2) ((uint32_t*)zero_row)[tid] = 0u;
    if (wave == 0) {
        const int first = lane < 32 ? tt[lane] : 0;
        const int c = lane < CT_TAPS ? tt[lane + 1] - first : 0;
        const int nc = (c + CH - 1) / CH;
        int x = nc;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) {
            const int y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        for (int j = 0; j < nc; ++j) {
            ch_tap[x - nc + j] = lane;
            ch_base[x - nc + j] = first + j * CH;
            ch_cnt[x - nc + j] = min(CH, c - j * CH);
        }
        if (lane == 31) n_chunks = x;
    }
    // the taps of the output voxels this lane holds as MFMA columns, and their sums (start: the bias)
    uint32_t taps_of[GPW];
    f32x16 acc[GPW];
#pragma unroll
    for (int gi = 0; gi < GPW; ++gi) {
        const int o = (pw * GPW + gi) * 32 + col;
        taps_of[gi] = o < nv ? vox_taps[v0 + o] : 0u;
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[gi][v] = bias ? (float)bias[cout0 + 32 * cw + 8 * (v / 4) + 4 * hf + v % 4] : 0.f;
    }
    __syncthreads();
    const int nch = n_chunks;   // >= 1: every voxel pairs with itself

    // ---- a ring of DEPTH chunks in flight: the weights of the chunk's tap (this wave's 32 output
    // channels) and the chunk's input rows, both as registers. Every load is unconditional (chunks
    // past the end repeat the last one, rows past a chunk's count repeat its first row), so the
    // number of loads in flight is fixed and a wait for one chunk leaves the younger ones in flight.
    struct Slot {
        u32x4 w[KS];
        u32x4 g[NL];
        uint32_t word[NL];
    };
    Slot ring[DEPTH];
    const T* wbase = packed_w + ((int64_t)(cout0 / 32 + cw) * KS * 64 + lane) * 8;
    constexpr int64_t W_TAP = (int64_t)(C / 32) * KS * 64 * 8;   // halfs per tap
    auto issue = [&](int k, Slot& s) {
        k = min(k, nch - 1);
        const int t = ch_tap[k], base = ch_base[k], count = ch_cnt[k];
#pragma unroll
        for (int i = 0; i < KS; ++i) s.w[i] = *(const u32x4*)(wbase + t * W_TAP + (int64_t)i * 64 * 8);
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int row = i * RPP + tid / LPR;
            s.word[i] = plist[base + (row < count ? row : 0)];
            s.g[i] = *(const u32x4*)(feat + (int64_t)(s.word[i] & CT_IN_MASK) * C + (tid % LPR) * 8);
        }
    };
    auto stage = [&](int k, const Slot& s) {
        const int count = ch_cnt[min(k, nch - 1)];
        T* xb = xs + (size_t)(k & 1) * TV * C;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int row = i * RPP + tid / LPR;
            if (row < count) *(u32x4*)(xb + swz<C>((int)(s.word[i] >> 24), tid % LPR)) = s.g[i];
        }
    };
    auto multiply = [&](int k, const Slot& s) {
        if (k >= nch) return;
        const int t = ch_tap[k], base = ch_base[k], count = ch_cnt[k];
        const int lo = (int)(plist[base] >> 24), hi = (int)(plist[base + count - 1] >> 24);   // outputs ascend inside a tap
        const T* xb = xs + (size_t)(k & 1) * TV * C;
#pragma unroll
        for (int gi = 0; gi < GPW; ++gi) {
            const int g = pw * GPW + gi;
            if (g * 32 + 31 >= lo && g * 32 <= hi) {   // uniform: the chunk has outputs in this group
                const int o = g * 32 + col;
                const bool present = ((taps_of[gi] >> t) & 1u) && o >= lo && o <= hi;
                if (__ballot(present) == 0) continue;   // none of the group's outputs has this tap
                // an absent neighbour reads the row of zeros: no branch, no registers to clear
                const T* row = present ? xb + o * C : zero_row;
                const int sw = present ? (o & 7) : 0;
#pragma unroll
                for (int i = 0; i < KS; ++i) {
                    const u32x4 x = *(const u32x4*)(row + (((2 * i + hf) ^ sw) * 8));
                    acc[gi] = TileOps<T>::mfma(__builtin_bit_cast(v8, s.w[i]), __builtin_bit_cast(v8, x), acc[gi]);
                }
            }
        }
    };

#pragma unroll
    for (int j = 0; j < DEPTH; ++j) issue(j, ring[j]);
    stage(0, ring[0]);
    __syncthreads();
    for (int k0 = 0; k0 < nch; k0 += DEPTH) {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            // no branch around the loads: past the end nothing is multiplied and the last chunk is staged again
            const int k = k0 + j;
            multiply(k, ring[j]);
            stage(k + 1, ring[(j + 1) % DEPTH]);
            __syncthreads();
            issue(k + DEPTH, ring[j]);
        }
    }

    // ---- sums -> halfs in LDS by output row -> out, 16 bytes per lane
    // acc[gi][v]: output channel 32 cw + 8 (v / 4) + 4 hf + v % 4 of output voxel (pw GPW + gi) 32 + col
    T* ob = xs;   // [TV][COUT_WG + 8]
    constexpr int OS = COUT_WG + 8;
    static_assert((size_t)TV * OS * 2 <= 2 * S::XBUF, "output staging fits in the input buffers");
#pragma unroll
    for (int gi = 0; gi < GPW; ++gi) {
        const int o = (pw * GPW + gi) * 32 + col;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t p0 = TileOps<T>::pack2(acc[gi][4 * q], acc[gi][4 * q + 1]);
            const uint32_t p1 = TileOps<T>::pack2(acc[gi][4 * q + 2], acc[gi][4 * q + 3]);
            uint32_t* dst = (uint32_t*)(ob + o * OS + 32 * cw + 8 * q + 4 * hf);
            dst[0] = p0;
            dst[1] = p1;
        }
    }
    __syncthreads();
    for (int e = tid; e < nv * (COUT_WG / 8); e += THREADS) {
        const int r = e / (COUT_WG / 8), c8 = e % (COUT_WG / 8);
        *(u32x4*)(out + (v0 + r) * C + cout0 + c8 * 8) = *(const u32x4*)(ob + r * OS + c8 * 8);
    }
}

template <typename T, int C, int TV_ = CT_TV>
int launch_tiles(const void* feat, int64_t n, const void* packed_w, const void* bias, const int32_t* tile_tap,
                 const uint32_t* tile_pair, const uint32_t* vox_taps, void* out, hipStream_t stream) {
    typedef TileShape<C, TV_> S;
    auto kern = conv_tile_kernel<T, C, TV_>;
    static LdsGrant grant_attr_set;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, S::LDS, grant_attr_set)) return rc_;
    const dim3 grid((unsigned)ptv3_ceil_div(n, S::TV), (unsigned)(C / S::COUT_WG));
    hipLaunchKernelGGL(kern, grid, dim3(S::THREADS), S::LDS, stream, (const T*)feat, n, (const T*)packed_w,
                       (const T*)bias, tile_tap, tile_pair, vox_taps, (T*)out);
    PTV3_RETURN_LAUNCH();
}

template <typename T>
int dispatch_tiles(const void* feat, int64_t n, int c, int tile_voxels, const void* packed_w, const void* bias,
                   const int32_t* tile_tap, const uint32_t* tile_pair, const uint32_t* vox_taps, void* out,
                   hipStream_t stream) {
    if (c == 64 && tile_voxels == 128)
        return launch_tiles<T, 64>(feat, n, packed_w, bias, tile_tap, tile_pair, vox_taps, out, stream);
    if (c == 128 && tile_voxels == 128)
        return launch_tiles<T, 128>(feat, n, packed_w, bias, tile_tap, tile_pair, vox_taps, out, stream);
    if (c == 128 && tile_voxels == 96)
        return launch_tiles<T, 128, 96>(feat, n, packed_w, bias, tile_tap, tile_pair, vox_taps, out, stream);
    return PTV3_ESHAPE;
}

}  // namespace

extern "C" int ptv3_conv_plan_slots(const int32_t* tap_ptr, int taps, const int32_t* pair_in, const int32_t* pair_slot,
                                    int64_t n_pairs, int32_t* slot_pair, void* stream_) {
    if (taps < 1 || taps > 128 || n_pairs < 0) return PTV3_EINVAL;
    if (n_pairs == 0) return PTV3_OK;
    if (!tap_ptr || !pair_in || !pair_slot || !slot_pair) return PTV3_EINVAL;
    hipLaunchKernelGGL(plan_slots_kernel, dim3((unsigned)ptv3_ceil_div(n_pairs, CT_THREADS)), dim3(CT_THREADS), 0,
                       (hipStream_t)stream_, tap_ptr, taps, pair_in, pair_slot, n_pairs, slot_pair);
    PTV3_RETURN_LAUNCH();
}

extern "C" int64_t ptv3_conv_plan_tile_count(int64_t n) { return n < 0 ? 0 : ptv3_ceil_div(n, CT_TV); }

extern "C" int64_t ptv3_conv_plan_tile_count_sized(int64_t n, int tile_voxels) {
    return (n < 0 || (tile_voxels != 96 && tile_voxels != 128)) ? 0 : ptv3_ceil_div(n, tile_voxels);
}

extern "C" int ptv3_conv_plan_tiles_sized(const int32_t* row_ptr, const int32_t* slot_pair, int64_t n, int taps,
                                          int tile_voxels, int32_t* tile_tap, int32_t* tile_pair, int32_t* vox_taps,
                                          void* stream_) {
    if (n < 0 || n >= (1ll << 24)) return PTV3_EINVAL;
    if (taps != CT_TAPS || (tile_voxels != 96 && tile_voxels != 128)) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!row_ptr || !slot_pair || !tile_tap || !tile_pair || !vox_taps) return PTV3_EINVAL;
    hipLaunchKernelGGL(plan_tiles_kernel, dim3((unsigned)ptv3_ceil_div(n, tile_voxels)), dim3(tile_voxels), 0,
                       (hipStream_t)stream_, row_ptr, slot_pair, n, tile_tap, (uint32_t*)tile_pair, (uint32_t*)vox_taps);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_conv_plan_tiles(const int32_t* row_ptr, const int32_t* slot_pair, int64_t n, int taps,
                                    int32_t* tile_tap, int32_t* tile_pair, int32_t* vox_taps, void* stream_) {
    return ptv3_conv_plan_tiles_sized(row_ptr, slot_pair, n, taps, CT_TV, tile_tap, tile_pair, vox_taps, stream_);
}

extern "C" int ptv3_subm_conv_pack_weight(const void* weight, int dtype, int channels, int taps, void* packed,
                                          void* stream_) {
    if (channels < 32 || channels % 32 != 0 || taps < 1) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (!weight || !packed) return PTV3_EINVAL;
    const int64_t total = (int64_t)taps * channels * channels / 8;
    const dim3 grid((unsigned)ptv3_ceil_div(total, CT_THREADS));
    // both half types are 16-bit patterns here: one instantiation moves either
    hipLaunchKernelGGL(pack_weight_kernel<_Float16>, grid, dim3(CT_THREADS), 0, (hipStream_t)stream_,
                       (const _Float16*)weight, channels, taps, (_Float16*)packed);
    PTV3_RETURN_LAUNCH();
}

extern "C" int64_t ptv3_subm_conv_pack_weight_blocks(int channels, int taps) {
    if (channels < 32 || channels % 32 != 0 || taps < 1) return 0;
    return ptv3_ceil_div((int64_t)taps * channels * channels / 8, CT_THREADS);
}

extern "C" int ptv3_subm_conv_pack_weight_batch(const ptv3_pack_job* jobs, int n_jobs, int64_t n_blocks, void* stream_) {
    if (n_jobs < 0 || n_blocks < 0 || n_blocks > 0x7fffffffLL) return PTV3_EINVAL;
    if (n_jobs == 0 || n_blocks == 0) return PTV3_OK;
    if (!jobs) return PTV3_EINVAL;
    hipLaunchKernelGGL(pack_weight_batch_kernel, dim3((unsigned)n_blocks), dim3(CT_THREADS), 0, (hipStream_t)stream_, jobs,
                       n_jobs);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_subm_conv_tiles_fwd(const void* feat, int dtype, int64_t n, int channels, int taps,
                                        const void* packed_weight, const void* bias, const int32_t* tile_tap,
                                        const int32_t* tile_pair, const int32_t* vox_taps, void* out, void* stream_) {
    return ptv3_subm_conv_tiles_fwd_sized(feat, dtype, n, channels, taps, CT_TV, packed_weight, bias, tile_tap, tile_pair,
                                          vox_taps, out, stream_);
}

extern "C" int ptv3_subm_conv_tiles_fwd_sized(const void* feat, int dtype, int64_t n, int channels, int taps,
                                              int tile_voxels, const void* packed_weight, const void* bias,
                                              const int32_t* tile_tap, const int32_t* tile_pair, const int32_t* vox_taps,
                                              void* out, void* stream_) {
    if (n < 0 || n >= (1ll << 24)) return PTV3_EINVAL;
    if (taps != CT_TAPS) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (channels != 64 && channels != 128) return PTV3_ESHAPE;
    if (tile_voxels != 128 && !(tile_voxels == 96 && channels == 128)) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!feat || !packed_weight || !tile_tap || !tile_pair || !vox_taps || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const uint32_t *tp = (const uint32_t*)tile_pair, *vt = (const uint32_t*)vox_taps;
    if (dtype == PTV3_F16)
        return dispatch_tiles<_Float16>(feat, n, channels, tile_voxels, packed_weight, bias, tile_tap, tp, vt, out, stream);
    return dispatch_tiles<__bf16>(feat, n, channels, tile_voxels, packed_weight, bias, tile_tap, tp, vt, out, stream);
}
