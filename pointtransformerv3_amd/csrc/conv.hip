// Submanifold sparse convolution forward over the neighbour map, in two forms.
//
// Replaces spconv.SubMConv3d.forward at the reference call sites model.py:546-552 (xCPE,
// 3x3x3, bias) and :767-774 (stem, 5x5x5, no bias).
//
// Dense form (ptv3_subm_conv_fwd): output-stationary implicit GEMM. A work-group keeps a block
// of the output in MFMA accumulators over all taps, so every output element is written once and
// nothing is atomic; it pays MFMA work for every (voxel, tap) of the taps it visits. Best when a
// good part of the taps is occupied (deep levels of a scan: 35-50 %).
// Pair form (ptv3_subm_conv_pairs_fwd): rows of the GEMM are the ACTIVE (input, output) pairs,
// grouped by tap, so every MFMA column is real work whatever the sparsity (a 2 cm surface scan
// has 2-5 of 27 taps per voxel); one product row per pair goes to a scratch matrix and a segment
// sum per voxel finishes. Costs a round trip of that matrix; best for sparse maps, thin channels.
//
// Both take the product transposed (rows = output channels, columns = voxels / pairs) with
// v_mfma_f32_32x32x16: a lane's operand is then 8 consecutive input channels of one row, and its
// results are 4 consecutive output channels of one row. Global traffic moves in whole row
// segments (several lanes x 16 B per row) and a small wave-private LDS buffer converts between
// that shape and the one-row-per-lane operand layout: touching 8-16 lines per memory instruction
// instead of 32 is what keeps the address path from bounding the kernels.
// fp32: one thread per output element, plain FMA (parity path, not tuned).
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct HalfOps;
template <> struct HalfOps<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    }
    static __device__ __forceinline__ float to_float(_Float16 v) { return (float)v; }
};
template <> struct HalfOps<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    static __device__ __forceinline__ float to_float(__bf16 v) { return (float)v; }
};

constexpr int CONV_THREADS = 256;
constexpr int CONV_WAVES = CONV_THREADS / PTV3_WAVE;
constexpr int W_PAD = 8;           // halfs of padding per LDS weight row
constexpr int XS_STRIDE = 72;      // halfs per staged row (64 + 8 of padding against bank conflicts)

// The staging buffer is private to a wave and LDS operations of one wave execute in program
// order, so a write followed by a read of the same bytes needs no wait: only the compiler has
// to be kept from reordering the two.
__device__ __forceinline__ void lds_fence() { asm volatile("" ::: "memory"); }

// Dense output-stationary form. A work-group owns ROWS = 4 waves * MT * 32 voxels and
// COUT_TILE = NT * 32 output channels. One step is (tap, KC-channel slice): the
// W[couts, tap, slice] tile sits in LDS, double-buffered (the next tile is fetched into registers
// while this one is multiplied; one barrier per step); the neighbour rows of the step after are in
// flight as well, and the neighbour indices of the tap after next. Taps no voxel of the
// work-group has are skipped altogether; a wave skips the taps none of its voxels has.
//
// PAIRS == true turns the same kernel into a tile of the pair form: the work-group takes ROWS
// consecutive entries of ONE tap of the tap-major pair list (found from tap_ptr), its rows are
// pair_in[...], there is a single tap to visit, and product rows go to out[pair_slot[...]]
// without bias. Used where the weight-stationary pair kernel would need most of the LDS for the
// weights of one tap (256 and more input channels).
template <typename T, int MT, int NT, int KC, bool PAIRS>
__global__ __launch_bounds__(CONV_THREADS, 2) void subm_conv_dense_kernel(
    const T* __restrict__ feat, int64_t n, int cin, const int32_t* __restrict__ nbr, int taps,
    bool tap_major, const T* __restrict__ weight, const T* __restrict__ bias, int cout,
    T* __restrict__ out, const int32_t* __restrict__ pair_in, const int32_t* __restrict__ pair_slot,
    const int32_t* __restrict__ tap_ptr) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int ROWS = CONV_WAVES * MT * 32;
    constexpr int COUT_TILE = NT * 32;
    constexpr int W_PIECES = COUT_TILE * (KC / 8);                 // 16-byte pieces per weight tile
    constexpr int W_LOADS = (W_PIECES + CONV_THREADS - 1) / CONV_THREADS;
    constexpr int LPR = KC / 8;           // lanes per staged row segment
    constexpr int RPI = 64 / LPR;         // rows per gather instruction
    constexpr int ITS = 32 / RPI;         // gather instructions per 32-row group
    __shared__ __align__(16) T w_lds[2][COUT_TILE][KC + W_PAD];
    __shared__ __align__(16) T xs_all[CONV_WAVES][32 * XS_STRIDE];
    __shared__ uint32_t wg_mask[4];

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int srow = lane / LPR, spc = lane % LPR;
    T* xs = xs_all[wave];
    const int cout0 = blockIdx.y * COUT_TILE;
    // dense: first voxel of the wave. pairs: first row of the wave inside the tile
    const int64_t vox0 = (PAIRS ? 0 : (int64_t)blockIdx.x * ROWS) + wave * (MT * 32);
    // neighbour map entry (voxel i, tap t): voxel-major (n,taps) or tap-major (taps,n)
    auto nbr_at = [&](int64_t i, int t) { return tap_major ? nbr[(int64_t)t * n + i] : nbr[i * taps + t]; };

    int only_tap = -1, pstart = 0, pcount = 0;
    uint32_t mask[4] = {0, 0, 0, 0};
    if (PAIRS) {
        // which tap does tile blockIdx.x belong to? lane l looks at taps l and l+64 (taps <= 128)
        const int rid = blockIdx.x;
        int first[2], cnt[2], nr[2], incl[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int tt = lane + 64 * k;
            first[k] = tt < taps ? tap_ptr[tt] : 0;
            cnt[k] = tt < taps ? tap_ptr[tt + 1] - first[k] : 0;
            nr[k] = (cnt[k] + ROWS - 1) / ROWS;
        }
        int carry = 0;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int xsum = nr[k];
#pragma unroll
            for (int off = 1; off < PTV3_WAVE; off <<= 1) {
                const int v = __shfl_up(xsum, off, PTV3_WAVE);
                if (lane >= off) xsum += v;
            }
            incl[k] = xsum + carry;
            carry += __shfl(xsum, PTV3_WAVE - 1, PTV3_WAVE);
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint64_t hit = __ballot(nr[k] > 0 && rid < incl[k] && rid >= incl[k] - nr[k]);
            if (hit && only_tap < 0) {
                const int l = __ffsll((unsigned long long)hit) - 1;
                const int rel = rid - (__shfl(incl[k], l, PTV3_WAVE) - __shfl(nr[k], l, PTV3_WAVE));
                only_tap = 64 * k + l;
                pstart = __shfl(first[k], l, PTV3_WAVE) + rel * ROWS;
                pcount = min(ROWS, __shfl(cnt[k], l, PTV3_WAVE) - rel * ROWS);
            }
        }
        if (only_tap < 0) return;   // the grid is an upper bound on the number of tiles
    } else {
        // taps any voxel of the work-group has (bit t of a 128-bit mask)
        if (tid < 4) wg_mask[tid] = 0;
        __syncthreads();
        for (int t = 0; t < taps; ++t) {
            bool any = false;
#pragma unroll
            for (int a = 0; a < MT; ++a) {
                const int64_t v = vox0 + a * 32 + col;
                any |= hf == 0 && v < n && nbr_at(v, t) >= 0;
            }
            if (__ballot(any) != 0 && lane == 0) atomicOr(&wg_mask[t >> 5], 1u << (t & 31));
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; ++k) mask[k] = wg_mask[k];
    }
    // input rows of tap t in staging shape: lane (srow, spc) serves rows srow + RPI*it of each group
    auto load_src = [&](int t, int32_t (&src)[MT][ITS]) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int64_t v = vox0 + a * 32 + it * RPI + srow;
                if (PAIRS) src[a][it] = (t == only_tap && v < pcount) ? pair_in[pstart + v] : -1;
                else src[a][it] = (t < taps && v < n) ? nbr_at(v, t) : -1;
            }
    };
    auto next_tap = [&](int t) {
        if (PAIRS) return t < 0 ? only_tap : taps;
        ++t;
        while (t < taps && !((mask[t >> 5] >> (t & 31)) & 1u)) ++t;
        return t;
    };

    f32x16 acc[MT][NT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const int chunks = (cin + KC - 1) / KC;
    auto fetch_w = [&](int t, int c0, u32x4 (&wreg)[W_LOADS]) {
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int e = tid + i * CONV_THREADS;
            const int co = e / (KC / 8), pc = e % (KC / 8);
            u32x4 w = {0, 0, 0, 0};
            if (e < W_PIECES && cout0 + co < cout && c0 + pc * 8 < cin)
                w = *(const u32x4*)(weight + ((int64_t)(cout0 + co) * taps + t) * cin + c0 + pc * 8);
            wreg[i] = w;
        }
    };
    auto store_w = [&](int buf, const u32x4 (&wreg)[W_LOADS]) {
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int e = tid + i * CONV_THREADS;
            const int co = e / (KC / 8), pc = e % (KC / 8);
            if (e < W_PIECES) *(u32x4*)&w_lds[buf][co][pc * 8] = wreg[i];
        }
    };
    auto gather_raw = [&](const int32_t (&src)[MT][ITS], int c0, u32x4 (&raw)[MT][ITS]) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                raw[a][it] = (u32x4){0, 0, 0, 0};
                if (c0 + spc * 8 < cin && src[a][it] >= 0)
                    raw[a][it] = *(const u32x4*)(feat + (int64_t)src[a][it] * cin + c0 + spc * 8);
            }
    };
    auto wave_has = [&](const int32_t (&src)[MT][ITS]) {
        bool any = false;
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) any |= src[a][it] >= 0;
        return __ballot(any) != 0;
    };

    int t = next_tap(-1);
    int tn = t < taps ? next_tap(t) : taps;
    int chunk = 0, buf = 0;
    int32_t src_t[MT][ITS], src_tn[MT][ITS];
    u32x4 wreg[W_LOADS];
    u32x4 raw[MT][ITS];
    load_src(t, src_t);
    load_src(tn, src_tn);
    if (t < taps) {
        fetch_w(t, 0, wreg);
        gather_raw(src_t, 0, raw);
        store_w(0, wreg);
    }
    __syncthreads();
    while (t < taps) {
        const bool tap_ends = (chunk + 1 == chunks);
        const int t2 = tap_ends ? tn : t;
        const int chunk2 = tap_ends ? 0 : chunk + 1;
        const bool has_next = t2 < taps;
        const bool active = wave_has(src_t);
        // this step's rows: staging shape -> one row per lane
        u32x4 x[KC / 16][MT];
        if (active) {
#pragma unroll
            for (int a = 0; a < MT; ++a) {
#pragma unroll
                for (int it = 0; it < ITS; ++it) *(u32x4*)(xs + (it * RPI + srow) * XS_STRIDE + spc * 8) = raw[a][it];
                lds_fence();
#pragma unroll
                for (int ks = 0; ks < KC / 16; ++ks) x[ks][a] = *(const u32x4*)(xs + col * XS_STRIDE + ks * 16 + hf * 8);
                lds_fence();
            }
        }
        // the step after this one: weights, rows, and (at a tap boundary) indices two taps ahead
        int tnn = tn;
        int32_t src_tnn[MT][ITS];
        if (has_next) {
            fetch_w(t2, chunk2 * KC, wreg);
            if (tap_ends) gather_raw(src_tn, 0, raw);
            else gather_raw(src_t, chunk2 * KC, raw);
        }
        if (tap_ends) {
            tnn = has_next ? next_tap(tn) : taps;
            load_src(tnn, src_tnn);
        }
        if (active) {
#pragma unroll
            for (int ks = 0; ks < KC / 16; ++ks) {
                if (chunk * KC + ks * 16 < cin) {
#pragma unroll
                    for (int b = 0; b < NT; ++b) {
                        const v8 wfrag = __builtin_bit_cast(v8, *(const u32x4*)&w_lds[buf][b * 32 + col][ks * 16 + hf * 8]);
#pragma unroll
                        for (int a = 0; a < MT; ++a)
                            acc[a][b] = HalfOps<T>::mfma(wfrag, __builtin_bit_cast(v8, x[ks][a]), acc[a][b]);
                    }
                }
            }
        }
        if (has_next) store_w(buf ^ 1, wreg);
        __syncthreads();
        buf ^= 1;
        if (tap_ends) {
#pragma unroll
            for (int a = 0; a < MT; ++a)
#pragma unroll
                for (int it = 0; it < ITS; ++it) { src_t[a][it] = src_tn[a][it]; src_tn[a][it] = src_tnn[a][it]; }
            t = tn;
            tn = tnn;
        }
        chunk = chunk2;
    }

    // acc[a][b][v]: output channel cout0 + b*32 + 8*(v/4) + 4*hf + v%4 of voxel vox0 + a*32 + col.
    // Add the bias, go back to row-segment shape 64 channels at a time, store 16 bytes per lane.
#pragma unroll
    for (int a = 0; a < MT; ++a) {
#pragma unroll
        for (int b0 = 0; b0 < NT; b0 += 2) {
#pragma unroll
            for (int bb = 0; bb < 2 && b0 + bb < NT; ++bb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int b = b0 + bb;
                    const int co = cout0 + b * 32 + 8 * g + 4 * hf;
                    float r[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        r[q] = acc[a][b][4 * g + q] +
                               ((!PAIRS && bias && co + q < cout) ? HalfOps<T>::to_float(bias[co + q]) : 0.f);
                    u32x2 pk = {HalfOps<T>::pack2(r[0], r[1]), HalfOps<T>::pack2(r[2], r[3])};
                    *(u32x2*)(xs + col * XS_STRIDE + bb * 32 + 8 * g + 4 * hf) = pk;
                }
            lds_fence();
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int orow = it * 8 + (lane >> 3), opc = lane & 7;
                const int co = cout0 + b0 * 32 + opc * 8;
                const int64_t v = vox0 + a * 32 + orow;
                const u32x4 val = *(const u32x4*)(xs + orow * XS_STRIDE + opc * 8);
                int64_t dst = -1;
                if (PAIRS) { if (v < pcount) dst = pair_slot[pstart + v]; }
                else if (v < n) dst = v;
                if (dst >= 0 && co < cout && (NT - b0 >= 2 || opc < 4)) *(u32x4*)(out + dst * cout + co) = val;
            }
            lds_fence();
        }
    }
}

// Pair mode for wide inputs (cin a multiple of 32 * DEPTH), persistent work-groups.
// A tile is ROWS consecutive entries of ONE tap of the tap-major pair list times COUT_TILE output
// channels; the contraction runs in 32-channel steps. Both a step's MFMA work (a few hundred
// cycles) and a whole tile (cin / 32 steps) are short against the latency of the dependent loads
// that feed them (tap bounds -> pair indices -> input rows), so
//   * the input rows and the weight tile of the next DEPTH steps are in flight in a ring of
//     registers, and the ring runs on across tile boundaries: the last DEPTH steps of a tile
//     already fetch the first steps of the work-group's next tile;
//   * the pair indices of the next tile are fetched while this tile is multiplied;
//   * addresses are per-lane pointers set up once per tile (a step adds a constant), and the
//     loop body has no branches: rows past the end of a tile and output channels past cout read
//     a valid address and their products are never stored.
template <typename T, int MT, int NT, int DEPTH>
__global__ __launch_bounds__(CONV_THREADS, 2) void pair_gemm_kernel(
    const T* __restrict__ feat, int cin, int taps, const T* __restrict__ weight, int cout,
    T* __restrict__ y, const int32_t* __restrict__ pair_in, const int32_t* __restrict__ pair_slot,
    const int32_t* __restrict__ tap_ptr) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int KC = 32;
    constexpr int ROWS = CONV_WAVES * MT * 32;
    constexpr int COUT_TILE = NT * 32;
    constexpr int W_LOADS = COUT_TILE * (KC / 8) / CONV_THREADS;
    static_assert(W_LOADS >= 1 && COUT_TILE * (KC / 8) % CONV_THREADS == 0, "weight tile must split evenly");
    static_assert(DEPTH % 2 == 0, "the weight double buffer alternates with the ring");
    constexpr int LPR = KC / 8, RPI = 64 / LPR, ITS = 32 / RPI;
    __shared__ __align__(16) T w_lds[2][COUT_TILE][KC + W_PAD];
    __shared__ __align__(16) T xs_all[CONV_WAVES][32 * XS_STRIDE];

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int srow = lane / LPR, spc = lane % LPR;
    T* xs = xs_all[wave];
    const int row0 = wave * (MT * 32);   // first row of the wave inside a tile

    // Row tiles per tap, as an inclusive prefix over the taps: lane l holds taps l and l+64.
    int first[2], cnt[2], nr[2], incl[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int tt = lane + 64 * k;
        first[k] = tt < taps ? tap_ptr[tt] : 0;
        cnt[k] = tt < taps ? tap_ptr[tt + 1] - first[k] : 0;
        nr[k] = (cnt[k] + ROWS - 1) / ROWS;
    }
    int row_tiles = 0;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int xsum = nr[k];
#pragma unroll
        for (int off = 1; off < PTV3_WAVE; off <<= 1) {
            const int v = __shfl_up(xsum, off, PTV3_WAVE);
            if (lane >= off) xsum += v;
        }
        incl[k] = xsum + row_tiles;
        row_tiles += __shfl(xsum, PTV3_WAVE - 1, PTV3_WAVE);
    }
    const int col_tiles = (cout + COUT_TILE - 1) / COUT_TILE;
    const int total = row_tiles * col_tiles;
    if ((int)blockIdx.x >= total) return;

    struct Tile {
        const T* xptr[MT][ITS];   // input rows, staging shape: lane (srow, spc) serves rows srow + RPI*it
        const T* wptr[W_LOADS];   // weight pieces: thread e -> output channel e / 4, 8-channel piece e % 4
        int32_t slot[MT][4];      // y rows of the pairs this lane stores in the epilogue, -1 past the end
        int cout0;
    };
    auto setup = [&](int g_launch, Tile& tl) {
        // the column tiles of one row tile gather the same rows: same XCD (the grid is a multiple of 8 or a
        // single round), one after the other
        const int g = xcd_chunked_id(g_launch, total);
        const int rid = g / col_tiles;
        tl.cout0 = (g % col_tiles) * COUT_TILE;
        int tap = 0, pstart = 0, pcount = 1;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint64_t hit = __ballot(nr[k] > 0 && rid < incl[k] && rid >= incl[k] - nr[k]);
            if (hit) {
                const int l = __ffsll((unsigned long long)hit) - 1;
                const int rel = rid - (__shfl(incl[k], l, PTV3_WAVE) - __shfl(nr[k], l, PTV3_WAVE));
                tap = 64 * k + l;
                pstart = __shfl(first[k], l, PTV3_WAVE) + rel * ROWS;
                pcount = min(ROWS, __shfl(cnt[k], l, PTV3_WAVE) - rel * ROWS);
            }
        }
#pragma unroll
        for (int a = 0; a < MT; ++a) {
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int v = row0 + a * 32 + it * RPI + srow;
                const int32_t idx = pair_in[pstart + min(v, pcount - 1)];
                tl.xptr[a][it] = feat + (int64_t)idx * cin + spc * 8;
            }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int v = row0 + a * 32 + it * 8 + (lane >> 3);
                tl.slot[a][it] = v < pcount ? pair_slot[pstart + v] : -1;
            }
        }
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int e = tid + i * CONV_THREADS;
            const int co = min(tl.cout0 + e / (KC / 8), cout - 1), pc = e % (KC / 8);
            tl.wptr[i] = weight + ((int64_t)co * taps + tap) * cin + pc * 8;
        }
    };

    u32x4 raw[DEPTH][MT][ITS], wreg[DEPTH][W_LOADS];
    auto issue = [&](const Tile& tl, int step, u32x4 (&r)[MT][ITS], u32x4 (&w)[W_LOADS]) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) r[a][it] = *(const u32x4*)(tl.xptr[a][it] + step * KC);
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) w[i] = *(const u32x4*)(tl.wptr[i] + step * KC);
    };
    auto store_w = [&](int buf, const u32x4 (&w)[W_LOADS]) {
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int e = tid + i * CONV_THREADS;
            *(u32x4*)&w_lds[buf][e / (KC / 8)][(e % (KC / 8)) * 8] = w[i];
        }
    };
    f32x16 acc[MT][NT];
    // DEPTH steps starting at s0; afterwards the ring holds steps ahead .. ahead + DEPTH - 1 of `src`
    auto run_steps = [&](const Tile& src, int ahead) {
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            const int buf = j & 1;
            u32x4 x[KC / 16][MT];
#pragma unroll
            for (int a = 0; a < MT; ++a) {
#pragma unroll
                for (int it = 0; it < ITS; ++it) *(u32x4*)(xs + (it * RPI + srow) * XS_STRIDE + spc * 8) = raw[j][a][it];
                lds_fence();
#pragma unroll
                for (int ks = 0; ks < KC / 16; ++ks) x[ks][a] = *(const u32x4*)(xs + col * XS_STRIDE + ks * 16 + hf * 8);
                lds_fence();
            }
            store_w(buf ^ 1, wreg[(j + 1) % DEPTH]);   // weights of the step after this one
            issue(src, ahead + j, raw[j], wreg[j]);
            u32x4 wf[KC / 16][NT];
#pragma unroll
            for (int ks = 0; ks < KC / 16; ++ks)
#pragma unroll
                for (int b = 0; b < NT; ++b) wf[ks][b] = *(const u32x4*)&w_lds[buf][b * 32 + col][ks * 16 + hf * 8];
#pragma unroll
            for (int ks = 0; ks < KC / 16; ++ks)
#pragma unroll
                for (int b = 0; b < NT; ++b)
#pragma unroll
                    for (int a = 0; a < MT; ++a)
                        acc[a][b] = HalfOps<T>::mfma(__builtin_bit_cast(v8, wf[ks][b]), __builtin_bit_cast(v8, x[ks][a]), acc[a][b]);
            __syncthreads();
        }
    };

    const int steps = cin / KC;   // a multiple of DEPTH
    Tile cur, nxt;
    setup(blockIdx.x, cur);
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) issue(cur, j, raw[j], wreg[j]);
    store_w(0, wreg[0]);
    __syncthreads();

    for (int g = blockIdx.x; g < total; g += gridDim.x) {
        const int gn = g + (int)gridDim.x;
        setup(gn < total ? gn : g, nxt);   // without a next tile the ring re-reads this one (never used)
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
        for (int s0 = 0; s0 + DEPTH < steps; s0 += DEPTH) run_steps(cur, s0 + DEPTH);
        run_steps(nxt, 0);

        // acc[a][b][v]: output channel cout0 + b*32 + 8*(v/4) + 4*hf + v%4 of pair row0 + a*32 + col.
        // Back to row-segment shape 64 channels at a time, 16 bytes per lane to y[slot].
#pragma unroll
        for (int a = 0; a < MT; ++a) {
#pragma unroll
            for (int b0 = 0; b0 < NT; b0 += 2) {
#pragma unroll
                for (int bb = 0; bb < 2 && b0 + bb < NT; ++bb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int b = b0 + bb;
                        u32x2 pk = {HalfOps<T>::pack2(acc[a][b][4 * q], acc[a][b][4 * q + 1]),
                                    HalfOps<T>::pack2(acc[a][b][4 * q + 2], acc[a][b][4 * q + 3])};
                        *(u32x2*)(xs + col * XS_STRIDE + bb * 32 + 8 * q + 4 * hf) = pk;
                    }
                lds_fence();
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int orow = it * 8 + (lane >> 3), opc = lane & 7;
                    const int co = cur.cout0 + b0 * 32 + opc * 8;
                    const u32x4 val = *(const u32x4*)(xs + orow * XS_STRIDE + opc * 8);
                    if (cur.slot[a][it] >= 0 && co < cout && (NT - b0 >= 2 || opc < 4))
                        *(u32x4*)(y + (int64_t)cur.slot[a][it] * cout + co) = val;
                }
                lds_fence();
            }
        }
        cur = nxt;
    }
}

// Pair mode for 256-channel layers, weight-stationary in REGISTERS.
// A work-group takes one tap and a range of that tap's pairs. Its 8 waves are 2 row halves x 4 output-channel
// quarters; a wave keeps W[its 64 output channels, tap, all 256 input channels] as MFMA operand fragments in
// 128 registers for its whole life (staged once through LDS so that the global reads are whole rows), and the
// range streams through 64 pairs at a time. Inside the loop the only LDS traffic is the gathered input rows
// (0.5 KB per MFMA: every row fragment meets two weight fragments that are already in registers) and the only
// stream from memory is those rows; the weights leave L2 once per work-group instead of once per tile.
// The input rows of a tile go through LDS in 64-channel steps (64 rows x 128 B), double-buffered, one barrier per
// step, software-pipelined by hand: right after the barrier that publishes step s+1 a wave asks for its
// fragments of step s+1 and then issues the eight MFMAs of step s, so the LDS reads run under the matrix work
// instead of in front of it. The rows of the next four steps (a whole tile) are in flight in a ring of registers
// that runs on across tile boundaries; pair indices and result slots are fetched two and one tiles ahead.
// Product rows go to y[pair_slot] for the segment sum, as in the other pair kernels.
constexpr int WS_THREADS = 512;
constexpr int WS_ROWS = 64;
constexpr int WS_KC = 64;
constexpr int WS_XSTRIDE = WS_KC + 8;   // halfs per staged row
constexpr int WS_DEPTH = 4;
constexpr int WS_CIN = 256, WS_COUT = 256;

template <typename T>
__global__ __launch_bounds__(WS_THREADS, 2) void pair_wstat_kernel(
    const T* __restrict__ feat, int taps, const T* __restrict__ weight, int cout, T* __restrict__ y,
    const int32_t* __restrict__ pair_in, const int32_t* __restrict__ pair_slot, const int32_t* __restrict__ tap_ptr,
    int range_rows) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int CIN = WS_CIN, COUT_T = WS_COUT;
    constexpr int KSTEPS = CIN / WS_KC;        // 4
    constexpr int KS = WS_KC / 16;             // MFMA contraction steps per staged step
    constexpr int WSTRIDE = CIN + W_PAD;
    constexpr int NT = 2;
    constexpr int XBUF = WS_ROWS * WS_XSTRIDE;
    static_assert(KSTEPS % 2 == 0 && KSTEPS == WS_DEPTH, "buffer parity and ring position carry over from tile to tile");
    static_assert(WS_THREADS == WS_ROWS * (WS_KC / 8), "one 16-byte piece per thread and step");
    extern __shared__ __align__(16) unsigned char ws_smem[];
    T* w_lds = (T*)ws_smem;                       // [COUT_T][WSTRIDE], only while the fragments are taken
    T* x_lds = w_lds + COUT_T * WSTRIDE;          // [2][WS_ROWS][WS_XSTRIDE]

    // which (tap, range) is mine: ranges of range_rows pairs, tap after tap
    int g = blockIdx.x, tap = -1, p0 = 0, p1 = 0;
    for (int t = 0; t < taps; ++t) {
        const int first = tap_ptr[t], cnt = tap_ptr[t + 1] - first;
        const int nr = (cnt + range_rows - 1) / range_rows;
        if (g < nr) {
            tap = t;
            p0 = first + g * range_rows;
            p1 = min(first + cnt, p0 + range_rows);
            break;
        }
        g -= nr;
    }
    if (tap < 0) return;
    const int cout0 = blockIdx.y * COUT_T;
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int row0 = (wave >> 2) * 32;                 // the wave's first row inside a tile
    const int c0 = (wave & 3) * (NT * 32);             // its first output channel inside the tile
    const int grow = tid >> 3, gpc = tid & 7;          // the row and 16-byte piece this thread gathers

    const int n_tiles = (p1 - p0 + WS_ROWS - 1) / WS_ROWS;
    auto gather_ptr = [&](int tile) {
        const int v = p0 + min(tile, n_tiles - 1) * WS_ROWS + grow;
        return feat + (int64_t)pair_in[min(v, p1 - 1)] * CIN + gpc * 8;
    };
    const T* ptr_cur = gather_ptr(0);
    const T* ptr_nxt = gather_ptr(1);
    const T* ptr_nn = gather_ptr(2);
    u32x4 ring[WS_DEPTH];   // ring[r]: the earliest step not yet in LDS whose number is r modulo WS_DEPTH
#pragma unroll
    for (int j = 0; j < WS_DEPTH; ++j) ring[j] = *(const u32x4*)(ptr_cur + j * WS_KC);

    // ---- the tap's weights: whole rows into LDS, then this wave's fragments into registers
    {
        constexpr int PIECES = COUT_T * (CIN / 8) / WS_THREADS;   // 16 per thread, 8 in flight together
#pragma unroll
        for (int i0 = 0; i0 < PIECES; i0 += 8) {
            u32x4 piece[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * WS_THREADS, co = e / (CIN / 8), pc = e % (CIN / 8);
                piece[i] = *(const u32x4*)(weight + ((int64_t)(cout0 + co) * taps + tap) * CIN + pc * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * WS_THREADS, co = e / (CIN / 8), pc = e % (CIN / 8);
                *(u32x4*)(w_lds + co * WSTRIDE + pc * 8) = piece[i];
            }
        }
    }
    __syncthreads();
    u32x4 wreg[NT][CIN / 16];
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
        for (int k = 0; k < CIN / 16; ++k)
            wreg[b][k] = *(const u32x4*)(w_lds + (c0 + b * 32 + col) * WSTRIDE + k * 16 + hf * 8);

    const T* xa = x_lds + (row0 + col) * WS_XSTRIDE + hf * 8;
    T* xw = x_lds + grow * WS_XSTRIDE + gpc * 8;
    // where the product rows go: lane l holds the slot of the wave's row l % 32 (its 32 rows, in store order)
    int32_t slot_nxt = pair_slot[min(p0 + row0 + col, p1 - 1)];
    // nothing but the ring may be in flight when the loop is entered: the wait-count bookkeeping of a loop is
    // the union of its entry and its back edge, and a value still pending at entry would be waited for in every
    // iteration -- in issue order, i.e. together with the whole ring
    asm volatile("" ::"v"(slot_nxt));
    asm volatile("" ::"v"(ptr_nn));
    // the weight rows in LDS are dead once every wave holds its fragments (the first barrier below): each wave
    // turns its product tiles into row segments there
    T* stage = w_lds + wave * (32 * XS_STRIDE);

    // step 0 of the first tile: into buffer 0, its fragments into registers
    *(u32x4*)xw = ring[0];
    ring[0] = *(const u32x4*)ptr_nxt;   // step WS_DEPTH = step 0 of the second tile
    __syncthreads();
    u32x4 xf[2][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xf[0][ks] = *(const u32x4*)(xa + ks * 16);

    for (int tile = 0; tile < n_tiles; ++tile) {
        // the rows three tiles on (the ring already asks for the first step of the tile after next while this one
        // is multiplied), and where the next tile's product rows go
        // (asked for a tile ahead: a value used right after its load would make the wave wait for every older
        // load as well, the whole ring of gathered rows included)
        const int v3 = p0 + min(tile + 3, n_tiles - 1) * WS_ROWS + grow;
        int32_t idx3 = pair_in[min(v3, p1 - 1)];
        const int32_t slot = slot_nxt;
        const int32_t slot_ahead = pair_slot[min(p0 + min(tile + 1, n_tiles - 1) * WS_ROWS + row0 + col, p1 - 1)];
        f32x16 acc[NT];
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
#pragma unroll
        for (int kc = 0; kc < KSTEPS; ++kc) {
            // publish step kc + 1 (of the next tile when this is the tile's last step) ...
            const int nb = (kc + 1) & 1;
            *(u32x4*)(xw + nb * XBUF) = ring[(kc + 1) % WS_DEPTH];
            // ... and ask for the step that takes its place in the ring: step kc + 1 of the next tile
            if (kc + 1 < KSTEPS) ring[(kc + 1) % WS_DEPTH] = *(const u32x4*)(ptr_nxt + (kc + 1) * WS_KC);
            else ring[0] = *(const u32x4*)ptr_nn;
            __syncthreads();
            // fragments of step kc + 1 first, then the products of step kc
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) xf[nb][ks] = *(const u32x4*)(xa + nb * XBUF + ks * 16);
            __builtin_amdgcn_sched_barrier(0);   // the scheduler would put the reads behind the matrix work
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int b = 0; b < NT; ++b)
                    acc[b] = HalfOps<T>::mfma(__builtin_bit_cast(v8, wreg[b][kc * KS + ks]),
                                              __builtin_bit_cast(v8, xf[kc & 1][ks]), acc[b]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // acc[b][v]: output channel cout0 + c0 + b*32 + 8*(v/4) + 4*hf + v%4 of pair row0 + col.
        // Through the wave's own LDS rows into row-segment shape: a store instruction then writes 8 rows x 128 B
        // (8 lanes x 16 B per row) instead of 32 rows x 16 B.
        // Rows past the end of the range repeat its last pair (same input row, same slot): they store the same
        // values to the same place, so neither the loads nor the stores of the loop are conditional -- with a
        // branch around them the wait counts in front of the ring would be those of the path that skips them.
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                u32x2 pk = {HalfOps<T>::pack2(acc[b][4 * q], acc[b][4 * q + 1]),
                            HalfOps<T>::pack2(acc[b][4 * q + 2], acc[b][4 * q + 3])};
                *(u32x2*)(stage + col * XS_STRIDE + b * 32 + 8 * q + 4 * hf) = pk;
            }
        lds_fence();
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int orow = it * 8 + (lane >> 3), opc = lane & 7;
            const u32x4 val = *(const u32x4*)(stage + orow * XS_STRIDE + opc * 8);
            const int32_t dst = __shfl(slot, orow, PTV3_WAVE);
            *(u32x4*)(y + (int64_t)dst * cout + cout0 + c0 + opc * 8) = val;
        }
        lds_fence();
        ptr_cur = ptr_nxt;
        ptr_nxt = ptr_nn;
        // tied to the last product so that the index is not turned into a pointer (and waited for, with every
        // older load) at the top of the tile
        asm volatile("" : "+v"(idx3) : "v"(acc[NT - 1][15]));
        ptr_nn = feat + (int64_t)idx3 * CIN + gpc * 8;
        slot_nxt = slot_ahead;
    }
}

// Pair mode, weight-stationary. A work-group takes one tap and a range of up to `range_rows`
// of that tap's pairs (tap-major list), keeps W[couts, tap, all input channels] in LDS for its
// whole life and streams the range through it in tiles of ROWS pairs. Steps (tile, 64-channel
// slice) are software-pipelined: the input rows of step s+1 and the pair indices of the tile after
// next are in flight while the MFMAs of step s run; there is no block barrier after the weights
// are staged.
// Global traffic moves in whole 128-byte row segments: a gather instruction fetches 8 rows x 128 B
// (8 lanes x 16 B per row) and a result store writes 8 rows x 128 B; a small wave-private LDS
// buffer converts between that shape and the MFMA register layout (one row per lane). Touching 8
// lines per instruction instead of 32 is what keeps the address path from bounding the kernel.
// PKC: input channels per step (64, or 32 where the 128-register accumulator leaves no room for
// a 64-channel prefetch). A staged row segment is PKC*2 bytes = LPR lanes x 16 B.
template <typename T, int MT, int NT, int PKC>
__global__ __launch_bounds__(CONV_THREADS, 2) void subm_conv_pairs_kernel(
    const T* __restrict__ feat, int cin, int taps, const T* __restrict__ weight, int cout,
    T* __restrict__ y, const int32_t* __restrict__ pair_in, const int32_t* __restrict__ pair_slot,
    const int32_t* __restrict__ tap_ptr, int range_rows) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int ROWS = CONV_WAVES * MT * 32;
    constexpr int COUT_TILE = NT * 32;
    extern __shared__ __align__(16) unsigned char conv_smem[];
    const int w_stride = cin + W_PAD;
    T* w_lds = (T*)conv_smem;                                   // [COUT_TILE][cin + W_PAD]
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    T* xs = w_lds + (size_t)COUT_TILE * w_stride + (size_t)wave * (32 * XS_STRIDE);   // wave-private [32][72]
    const int col = lane & 31, hf = lane >> 5;
    constexpr int LPR = PKC / 8;          // lanes per staged row segment
    constexpr int RPI = 64 / LPR;         // rows per load/store instruction
    constexpr int ITS = 32 / RPI;         // instructions per 32-row group
    const int srow = lane / LPR, spc = lane % LPR;
    const int cout0 = blockIdx.y * COUT_TILE;

    // ---- which (tap, range) is blockIdx.x? ranges never straddle taps. Lane l looks at taps l
    // and l+64 (taps <= 128): one round of loads, then a wave prefix sum of range counts.
    int tap = -1, start = 0, count = 0;
    {
        const int rid = blockIdx.x;
        int first[2], cnt[2], nr[2], incl[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int tt = lane + 64 * k;
            first[k] = tt < taps ? tap_ptr[tt] : 0;
            cnt[k] = tt < taps ? tap_ptr[tt + 1] - first[k] : 0;
            nr[k] = (cnt[k] + range_rows - 1) / range_rows;
        }
        int carry = 0;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            int x = nr[k];
#pragma unroll
            for (int off = 1; off < PTV3_WAVE; off <<= 1) {
                const int v = __shfl_up(x, off, PTV3_WAVE);
                if (lane >= off) x += v;
            }
            incl[k] = x + carry;
            carry += __shfl(x, PTV3_WAVE - 1, PTV3_WAVE);
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint64_t hit = __ballot(nr[k] > 0 && rid < incl[k] && rid >= incl[k] - nr[k]);
            if (hit && tap < 0) {
                const int l = __ffsll((unsigned long long)hit) - 1;
                const int rel = rid - (__shfl(incl[k], l, PTV3_WAVE) - __shfl(nr[k], l, PTV3_WAVE));
                tap = 64 * k + l;
                start = __shfl(first[k], l, PTV3_WAVE) + rel * range_rows;
                count = min(range_rows, __shfl(cnt[k], l, PTV3_WAVE) - rel * range_rows);
            }
        }
    }
    if (tap < 0) return;   // the grid is an upper bound on the number of ranges

    // ---- stage W[cout0.., tap, :] once
    {
        const int pieces_per_row = cin / 8;
        for (int e = tid; e < COUT_TILE * pieces_per_row; e += CONV_THREADS) {
            const int co = e / pieces_per_row, pc = e % pieces_per_row;
            u32x4 w = {0, 0, 0, 0};
            if (cout0 + co < cout)
                w = *(const u32x4*)(weight + ((int64_t)(cout0 + co) * taps + tap) * cin + pc * 8);
            *(u32x4*)(w_lds + co * w_stride + pc * 8) = w;
        }
    }

    const int n_tiles = (count + ROWS - 1) / ROWS;
    const int chunks = (cin + PKC - 1) / PKC;
    const int wave_row0 = wave * (MT * 32);
    // pair indices in staging shape: lane (srow, spc) serves rows srow + 8*it of every 32-row group
    auto load_idx = [&](const int32_t* __restrict__ table, int tile, int32_t (&idx)[MT][ITS]) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int r = tile * ROWS + wave_row0 + a * 32 + it * RPI + srow;
                idx[a][it] = (tile < n_tiles && r < count) ? table[start + r] : -1;
            }
    };
    // 64-channel slice of 32 rows per group: 4 instructions of 8 rows x 128 B
    auto gather_raw = [&](const int32_t (&pin)[MT][ITS], int c0, u32x4 (&raw)[MT][ITS]) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                raw[a][it] = (u32x4){0, 0, 0, 0};
                if (c0 + spc * 8 < cin && pin[a][it] >= 0)
                    raw[a][it] = *(const u32x4*)(feat + (int64_t)pin[a][it] * cin + c0 + spc * 8);
            }
    };

    int32_t pin_c[MT][ITS], pin_n[MT][ITS];
    u32x4 raw[MT][ITS];
    load_idx(pair_in, 0, pin_c);
    load_idx(pair_in, 1, pin_n);
    gather_raw(pin_c, 0, raw);
    __syncthreads();   // weights staged

    f32x16 acc[MT][NT];
    for (int tile = 0; tile < n_tiles; ++tile) {
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
        // Narrow outputs (cin <= 64 in practice: one step per tile) fetch the input rows two tiles
        // ahead so that index load and gather never sit in the same step; wide ones have several
        // steps per tile to hide the index load and cannot spare the registers.
        constexpr bool DEEP = NT <= 2;
        int32_t pin_nn[MT][ITS], slot_c[MT][ITS];
        if (DEEP) load_idx(pair_in, tile + 2, pin_nn);
        for (int chunk = 0; chunk < chunks; ++chunk) {
            if (!DEEP && chunk == 0) load_idx(pair_in, tile + 1, pin_n);
            // output slots of this tile: needed after the last step's MFMAs
            if (chunk == chunks - 1) load_idx(pair_slot, tile, slot_c);
            // rows of this step: staging shape -> one row per lane, through the wave's LDS buffer
            u32x4 x[PKC / 16][MT];
#pragma unroll
            for (int a = 0; a < MT; ++a) {
#pragma unroll
                for (int it = 0; it < ITS; ++it) *(u32x4*)(xs + (it * RPI + srow) * XS_STRIDE + spc * 8) = raw[a][it];
                lds_fence();
#pragma unroll
                for (int ks = 0; ks < PKC / 16; ++ks) x[ks][a] = *(const u32x4*)(xs + col * XS_STRIDE + ks * 16 + hf * 8);
                lds_fence();
            }
            // next step's rows
            if (chunk + 1 < chunks) gather_raw(pin_c, (chunk + 1) * PKC, raw);
            else gather_raw(pin_n, 0, raw);   // first slice of the next tile (nothing past the end)
            const int c0 = chunk * PKC;
#pragma unroll
            for (int ks = 0; ks < PKC / 16; ++ks) {
                if (c0 + ks * 16 < cin) {
#pragma unroll
                    for (int b = 0; b < NT; ++b) {
                        const v8 wfrag = __builtin_bit_cast(
                            v8, *(const u32x4*)(w_lds + (b * 32 + col) * w_stride + c0 + ks * 16 + hf * 8));
#pragma unroll
                        for (int a = 0; a < MT; ++a)
                            acc[a][b] = HalfOps<T>::mfma(wfrag, __builtin_bit_cast(v8, x[ks][a]), acc[a][b]);
                    }
                }
                // keep the scheduler from hoisting every weight fragment of the step up front
                // (that costs 16 registers per 16-channel sub-step)
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // acc[a][b][v]: output channel cout0 + b*32 + 8*(v/4) + 4*hf + v%4 of the lane's row.
        // Back to staging shape, 64 channels (two 32-channel tiles) at a time, then 16-byte stores.
#pragma unroll
        for (int a = 0; a < MT; ++a) {
#pragma unroll
            for (int b0 = 0; b0 < NT; b0 += 2) {
#pragma unroll
                for (int bb = 0; bb < 2 && b0 + bb < NT; ++bb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int b = b0 + bb;
                        u32x2 pk = {HalfOps<T>::pack2(acc[a][b][4 * g], acc[a][b][4 * g + 1]),
                                    HalfOps<T>::pack2(acc[a][b][4 * g + 2], acc[a][b][4 * g + 3])};
                        *(u32x2*)(xs + col * XS_STRIDE + bb * 32 + 8 * g + 4 * hf) = pk;
                    }
                lds_fence();
                // 64 output channels of 32 rows = 8 lanes x 16 B per row, 8 rows per store
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    const int orow = it * 8 + (lane >> 3), opc = lane & 7;
                    const int co = cout0 + b0 * 32 + opc * 8;
                    const u32x4 v = *(const u32x4*)(xs + orow * XS_STRIDE + opc * 8);
                    // the slot of row `orow` sits in the lane that staged it: group (it*8)/RPI, lane
                    // (row within the group) * LPR
                    const int32_t slot = __shfl(slot_c[a][(it * 8) / RPI], (((it * 8) % RPI) + (lane >> 3)) * LPR, PTV3_WAVE);
                    if (slot >= 0 && co < cout && (NT - b0 >= 2 || opc < 4))
                        *(u32x4*)(y + (int64_t)slot * cout + co) = v;
                }
                lds_fence();
            }
        }
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                pin_c[a][it] = pin_n[a][it];
                if (DEEP) pin_n[a][it] = pin_nn[a][it];
            }
    }
}

// y (n_pairs, cout) in output-major slot order -> out[i] = bias + sum of voxel i's slots
template <typename T>
__global__ __launch_bounds__(256) void pair_segment_sum_kernel(const T* __restrict__ y,
                                                               const int32_t* __restrict__ row_ptr,
                                                               int64_t n, int cout,
                                                               const T* __restrict__ bias,
                                                               T* __restrict__ out) {
    typedef typename HalfOps<T>::v8 v8;
    const int groups = cout / 8;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * groups) return;
    const int64_t i = e / groups;
    const int c = (int)(e - i * groups) * 8;
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = bias ? HalfOps<T>::to_float(bias[c + k]) : 0.f;
    const int s0 = row_ptr[i], s1 = row_ptr[i + 1];
    // four rows in flight per thread; the additions keep the order s0, s0+1, ...
    const T* src = y + (int64_t)s0 * cout + c;
    for (int s = s0; s < s1; s += 4, src += 4 * (int64_t)cout) {
        u32x4 raw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            raw[j] = (u32x4){0, 0, 0, 0};
            if (s + j < s1) raw[j] = *(const u32x4*)(src + (int64_t)j * cout);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (s + j < s1) {
                const v8 v = __builtin_bit_cast(v8, raw[j]);
#pragma unroll
                for (int k = 0; k < 8; ++k) acc[k] += (float)v[k];
            }
        }
    }
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = HalfOps<T>::pack2(acc[2 * k], acc[2 * k + 1]);
    *(u32x4*)(out + i * cout + c) = r;
}

// fp32: one thread per (voxel, output channel); a wave shares the voxel when cout >= 64.
__global__ __launch_bounds__(256) void subm_conv_f32_kernel(
    const float* __restrict__ feat, int64_t n, int cin, const int32_t* __restrict__ nbr, int taps,
    bool tap_major, const float* __restrict__ weight, const float* __restrict__ bias, int cout,
    float* __restrict__ out) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n * cout) return;
    const int64_t i = e / cout;
    const int co = (int)(e - i * cout);
    float acc = bias ? bias[co] : 0.f;
    for (int t = 0; t < taps; ++t) {
        const int32_t src = tap_major ? nbr[(int64_t)t * n + i] : nbr[i * taps + t];
        if (src < 0) continue;
        const float* x = feat + (int64_t)src * cin;
        const float* w = weight + ((int64_t)co * taps + t) * cin;
        float part = 0.f;
        for (int c = 0; c < cin; ++c) part = fmaf(x[c], w[c], part);
        acc += part;
    }
    out[e] = acc;
}

template <typename T, int MT, int NT>
void launch_dense(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps, bool tap_major,
                  const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    constexpr int KC = NT >= 4 ? 32 : 64;   // the 128-register accumulator leaves room for 32-channel prefetches only
    dim3 grid((unsigned)ptv3_ceil_div(n, ROWS), (unsigned)ptv3_ceil_div(cout, COUT_TILE));
    hipLaunchKernelGGL((subm_conv_dense_kernel<T, MT, NT, KC, false>), grid, dim3(CONV_THREADS), 0, stream,
                       (const T*)feat, n, cin, nbr, taps, tap_major, (const T*)weight, (const T*)bias, cout, (T*)out,
                       (const int32_t*)nullptr, (const int32_t*)nullptr, (const int32_t*)nullptr);
}

template <typename T>
void dispatch_dense(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps, bool tap_major,
                    const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    // Rows per work-group: 256 while that still yields about two work-groups per CU, else 128.
    const int64_t col_tiles = cout <= 64 ? 1 : ptv3_ceil_div(cout, 128);
    const bool wide = ptv3_ceil_div(n, 256) * col_tiles >= 512;
#define PTV3_DENSE(MT, NT) launch_dense<T, MT, NT>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream)
    if (cout <= 32) { if (wide) PTV3_DENSE(2, 1); else PTV3_DENSE(1, 1); }
    else if (cout <= 64) { if (wide) PTV3_DENSE(2, 2); else PTV3_DENSE(1, 2); }
    else { if (wide) PTV3_DENSE(2, 4); else PTV3_DENSE(1, 4); }
#undef PTV3_DENSE
}

template <typename T, int MT, int NT>
int launch_pairs(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                 const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                 hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    const size_t lds = ((size_t)COUT_TILE * (cin + W_PAD) + (size_t)CONV_WAVES * 32 * XS_STRIDE) * sizeof(T);
    if (lds > 160 * 1024) return PTV3_ESHAPE;
    auto kern = subm_conv_pairs_kernel<T, MT, NT, (NT >= 4 ? 32 : 64)>;
    static LdsGrant grant_lds_allowed;   // per instantiation and device; raised monotonically
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_lds_allowed)) return rc_;
    // Rows per work-group: long enough to amortise staging the weights, short enough to give
    // every CU a few work-groups.
    const int64_t col_tiles = ptv3_ceil_div(cout, COUT_TILE);
    int64_t range_rows = ROWS * 8;
    while (range_rows > ROWS && (n_pairs / range_rows + taps) * col_tiles < 1024) range_rows /= 2;
    dim3 grid((unsigned)(n_pairs / range_rows + taps), (unsigned)col_tiles);   // every tap may end with a partial range
    hipLaunchKernelGGL(kern, grid, dim3(CONV_THREADS), lds, stream, (const T*)feat, cin, taps, (const T*)weight, cout,
                       (T*)y, pair_in, pair_slot, tap_ptr, (int)range_rows);
    return PTV3_OK;
}

// pair tiles through the chunked kernel (55 KB of LDS whatever cin is)
template <typename T, int MT, int NT, int KC>
int launch_pairs_chunked_v(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                         const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                         hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    dim3 grid((unsigned)(n_pairs / ROWS + taps), (unsigned)ptv3_ceil_div(cout, COUT_TILE));
    hipLaunchKernelGGL((subm_conv_dense_kernel<T, MT, NT, KC, true>), grid, dim3(CONV_THREADS), 0, stream,
                       (const T*)feat, (int64_t)0, cin, (const int32_t*)nullptr, taps, false, (const T*)weight,
                       (const T*)nullptr, cout, (T*)y, pair_in, pair_slot, tap_ptr);
    return PTV3_OK;
}
template <typename T, int MT, int NT, int DEPTH>
int launch_pair_gemm(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                     const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                     hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    // persistent work-groups: as many as the machine holds at a time (or as there can be tiles)
    const int64_t tiles_max = (n_pairs / ROWS + taps) * ptv3_ceil_div(cout, COUT_TILE);
    const int64_t resident = 256 * 2;
    dim3 grid((unsigned)(tiles_max < resident ? tiles_max : resident));
    hipLaunchKernelGGL((pair_gemm_kernel<T, MT, NT, DEPTH>), grid, dim3(CONV_THREADS), 0, stream, (const T*)feat, cin,
                       taps, (const T*)weight, cout, (T*)y, pair_in, pair_slot, tap_ptr);
    return PTV3_OK;
}
template <typename T>
int launch_pair_wstat(const void* feat, int taps, int64_t n_pairs, const int32_t* tap_ptr, const int32_t* pair_in,
                      const int32_t* pair_slot, const void* weight, int cout, void* y, hipStream_t stream) {
    const size_t lds = ((size_t)WS_COUT * (WS_CIN + W_PAD) + 2 * (size_t)WS_ROWS * WS_XSTRIDE) * sizeof(T);
    static_assert(8 * 32 * XS_STRIDE <= WS_COUT * (WS_CIN + W_PAD), "the waves' staging rows fit where the weights were");
    auto kern = pair_wstat_kernel<T>;
    static LdsGrant grant_allowed;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_allowed)) return rc_;
    // One work-group per CU (its registers hold the weights). Ranges in whole tiles: one round of work-groups
    // over the machine, long enough to pay for staging one tap's weights.
    const int64_t col_tiles = cout / WS_COUT;
    int64_t range_rows = ptv3_ceil_div(ptv3_ceil_div(n_pairs * col_tiles, 256 - taps), WS_ROWS) * WS_ROWS;
    if (range_rows < 8 * WS_ROWS) range_rows = 8 * WS_ROWS;
    dim3 grid((unsigned)(n_pairs / range_rows + taps), (unsigned)col_tiles);   // every tap may end with a partial range
    hipLaunchKernelGGL(kern, grid, dim3(WS_THREADS), lds, stream, (const T*)feat, taps, (const T*)weight, cout, (T*)y,
                       pair_in, pair_slot, tap_ptr, (int)range_rows);
    return PTV3_OK;
}

template <typename T>
int launch_pairs_chunked(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                         const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                         hipStream_t stream) {
    // wide square-ish layers: one tap's weights stay in LDS
    if (cin == WS_CIN && cout % WS_COUT == 0 && taps <= 128)
        return launch_pair_wstat<T>(feat, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
    // the ring of the persistent kernel is four 32-channel steps deep
    if (cin % 128 == 0 && taps <= 128)
        return launch_pair_gemm<T, 1, 4, 4>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
    return launch_pairs_chunked_v<T, 2, 4, 32>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
}

template <typename T>
int dispatch_pairs(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                   const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                   hipStream_t stream) {
    // from 128 input channels on a tile is long enough (4+ contraction steps) for the persistent
    // tile kernel, which keeps more waves in flight than one tap's weights in LDS allow
    if (cin >= 128 && cout > 64)
        return launch_pairs_chunked<T>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
#define PTV3_PAIRS(MT, NT) return launch_pairs<T, MT, NT>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream)
    if (cout <= 32) PTV3_PAIRS(2, 1);
    if (cout <= 64) PTV3_PAIRS(2, 2);
    PTV3_PAIRS(2, 4);
#undef PTV3_PAIRS
}

}  // namespace

extern "C" int ptv3_subm_conv_fwd(const void* feat, int dtype, int64_t n, int cin,
                                  const int32_t* nbr, int taps, int tap_major_, const void* weight,
                                  const void* bias, int cout, void* out, void* stream_) {
    if (n < 0 || cin < 1 || cout < 1 || taps < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!feat || !nbr || !weight || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const bool tap_major = tap_major_ != 0;
    if (dtype == PTV3_F32) {
        hipLaunchKernelGGL(subm_conv_f32_kernel, dim3((unsigned)ptv3_ceil_div(n * cout, 256)), dim3(256),
                           0, stream, (const float*)feat, n, cin, nbr, taps, tap_major, (const float*)weight,
                           (const float*)bias, cout, (float*)out);
        PTV3_RETURN_LAUNCH();
    }
    // operand registers are 8-channel pieces of 16-channel steps; stores are 4-channel pieces
    if (cin % 16 != 0 || cout % 8 != 0) return PTV3_ESHAPE;
    if (dtype == PTV3_F16)
        dispatch_dense<_Float16>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
    else
        dispatch_dense<__bf16>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_subm_conv_pairs_fwd(const void* feat, int dtype, int64_t n, int cin, int taps,
                                        int64_t n_pairs, const int32_t* tap_ptr,
                                        const int32_t* row_ptr, const int32_t* pair_in,
                                        const int32_t* pair_slot, const void* weight,
                                        const void* bias, int cout, void* y, void* out,
                                        void* stream_) {
    if (n < 0 || cin < 1 || cout < 1 || taps < 1 || n_pairs < 0 || n_pairs >= (1ll << 31)) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;   // fp32 goes through ptv3_subm_conv_fwd
    if (cin % 16 != 0 || cout % 8 != 0) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!feat || !tap_ptr || !row_ptr || !weight || !out) return PTV3_EINVAL;
    if (n_pairs > 0 && (!pair_in || !pair_slot || !y)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const dim3 sgrid((unsigned)ptv3_ceil_div(n * (cout / 8), 256)), sblock(256);
    int rc = PTV3_OK;
    if (dtype == PTV3_F16) {
        if (n_pairs > 0)
            rc = dispatch_pairs<_Float16>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
        if (rc != PTV3_OK) return rc;
        hipLaunchKernelGGL(pair_segment_sum_kernel<_Float16>, sgrid, sblock, 0, stream, (const _Float16*)y,
                           row_ptr, n, cout, (const _Float16*)bias, (_Float16*)out);
    } else {
        if (n_pairs > 0)
            rc = dispatch_pairs<__bf16>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
        if (rc != PTV3_OK) return rc;
        hipLaunchKernelGGL(pair_segment_sum_kernel<__bf16>, sgrid, sblock, 0, stream, (const __bf16*)y, row_ptr,
                           n, cout, (const __bf16*)bias, (__bf16*)out);
    }
    PTV3_RETURN_LAUNCH();
}
