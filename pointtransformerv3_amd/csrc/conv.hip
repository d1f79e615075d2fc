// Submanifold sparse convolution forward as an output-stationary implicit GEMM over the
// neighbour map.
//
// Replaces spconv.SubMConv3d.forward at the reference call sites model.py:546-552 (xCPE,
// 3x3x3, bias) and :767-774 (stem, 5x5x5, no bias).
//
// Half-precision path: one GEMM core (below) keeps a block of the output in MFMA accumulators,
// stages weight tiles through double-buffered LDS and gathers neighbour rows straight into MFMA
// operand registers. The product is taken transposed (rows = output channels, columns = voxels)
// so a lane ends up holding 4 consecutive output channels of one voxel and stores 8 bytes.
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
constexpr int W_PAD = 8;         // halfs of padding per LDS weight row

// Shared GEMM core. A work-group owns ROWS = 4 waves * MT * 32 rows and COUT_TILE = NT * 32
// output channels; accumulators stay in registers. One "step" is (tap, 64-channel slice):
// the W[couts, tap, slice] tile sits in LDS (double-buffered: the next tile is fetched into
// registers while this one is multiplied), the rows' input features are gathered straight
// into MFMA operand registers (8 consecutive channels of one row = one 16-byte load).
//
// PAIRS == false: dense output-stationary mode. Row r is voxel row0 + r; for tap t its
//   input row is nbr[voxel][t] (or nothing); all taps accumulate into the same registers and
//   the voxel's output row is written once, with bias.
// PAIRS == true: a work-group processes up to ROWS consecutive entries of a tap-major list of
//   active (input row, output slot) pairs, all of ONE tap (tiles never straddle taps; the tap
//   is found from tap_ptr), and writes one product row per pair to y[slot]; a segment sum over
//   each voxel's slots finishes the convolution. Every MFMA column is a real pair, so the
//   matrix work is proportional to the active pairs, not to taps * voxels.
// KC: input channels per step (one LDS weight tile).
template <typename T, int MT, int NT, int KC, bool PAIRS>
__global__ __launch_bounds__(CONV_THREADS, 2) void subm_conv_gemm_kernel(
    const T* __restrict__ feat, int64_t n, int cin, const int32_t* __restrict__ nbr, int taps,
    bool tap_major, const T* __restrict__ weight, const T* __restrict__ bias, int cout,
    T* __restrict__ out, const int32_t* __restrict__ pair_in, const int32_t* __restrict__ pair_slot,
    const int32_t* __restrict__ tap_ptr) {
    typedef typename HalfOps<T>::v8 v8;
    constexpr int ROWS = CONV_WAVES * MT * 32;
    constexpr int COUT_TILE = NT * 32;
    constexpr int W_PIECES = COUT_TILE * (KC / 8);                 // 16-byte pieces per weight tile
    constexpr int W_LOADS = (W_PIECES + CONV_THREADS - 1) / CONV_THREADS;
    __shared__ __align__(16) T w_lds[2][COUT_TILE][KC + W_PAD];
    __shared__ uint32_t wg_mask;

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int cout0 = blockIdx.y * COUT_TILE;
    // neighbour map entry (voxel i, tap t): voxel-major (n,taps) or tap-major (taps,n)
    auto nbr_at = [&](int64_t i, int t) { return tap_major ? nbr[(int64_t)t * n + i] : nbr[i * taps + t]; };

    // ---- rows of this wave
    int64_t row[MT];      // dense: voxel id; pairs: index into the pair list (or -1)
    int32_t pin[MT];      // pairs: input row
    int only_tap = 0;
    uint32_t my_mask = 0;
    if (PAIRS) {
        // which tap does tile blockIdx.x belong to? tiles never straddle taps
        int tile = blockIdx.x, start = 0, count = 0;
        only_tap = -1;
        for (int tt = 0; tt < taps; ++tt) {
            const int first = tap_ptr[tt], cnt = tap_ptr[tt + 1] - first;
            const int tiles_here = (cnt + ROWS - 1) / ROWS;
            if (tile < tiles_here) {
                only_tap = tt;
                start = first + tile * ROWS;
                count = min(ROWS, cnt - tile * ROWS);
                break;
            }
            tile -= tiles_here;
        }
        if (only_tap < 0) return;   // grid is an upper bound on the number of tiles
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            const int r = wave * (MT * 32) + a * 32 + col;
            row[a] = r < count ? (int64_t)start + r : -1;
            pin[a] = row[a] >= 0 ? pair_in[row[a]] : -1;
        }
    } else {
        const int64_t row0 = (int64_t)blockIdx.x * ROWS + wave * (MT * 32);
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            row[a] = row0 + a * 32 + col;
            pin[a] = -1;
        }
        // taps any voxel of the work-group has: the others are skipped altogether
        if (tid == 0) wg_mask = 0;
        __syncthreads();
        for (int t = 0; t < taps && taps <= 32; ++t) {
            bool any = false;
#pragma unroll
            for (int a = 0; a < MT; ++a) any |= row[a] < n && nbr_at(row[a], t) >= 0;
            if (__ballot(any) != 0) my_mask |= 1u << (t & 31);
        }
        // 27 taps fit one word; for 125 taps (stem) the mask is not used: all taps are visited
        if (taps <= 32 && lane == 0) atomicOr(&wg_mask, my_mask);
        __syncthreads();
    }
    const uint32_t tap_mask = (PAIRS || taps > 32) ? 0xffffffffu : wg_mask;

    f32x16 acc[MT][NT];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const int chunks = (cin + KC - 1) / KC;
    // next active tap after t (pairs mode has exactly one)
    auto next_tap = [&](int t) {
        if (PAIRS) return t < 0 ? only_tap : taps;
        ++t;
        while (t < taps && taps <= 32 && !((tap_mask >> t) & 1u)) ++t;
        return t;
    };
    auto load_src = [&](int t, int32_t (&src)[MT]) {
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            if (PAIRS) src[a] = pin[a];
            else src[a] = (t < taps && row[a] < n) ? nbr_at(row[a], t) : -1;
        }
    };
    // global -> register fetch of one weight tile / of the rows' input slices
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
    auto gather_x = [&](const int32_t (&src)[MT], int c0, u32x4 (&x)[KC / 16][MT]) {
#pragma unroll
        for (int ks = 0; ks < KC / 16; ++ks)
#pragma unroll
            for (int a = 0; a < MT; ++a) {
                x[ks][a] = (u32x4){0, 0, 0, 0};
                if (c0 + ks * 16 < cin && src[a] >= 0)
                    x[ks][a] = *(const u32x4*)(feat + (int64_t)src[a] * cin + c0 + ks * 16 + hf * 8);
            }
    };

    // Pipeline: while the MFMAs of step s run, the weight tile and the gathered rows of step
    // s+1 are in flight, and the neighbour indices of the tap after next are being fetched.
    int t = next_tap(-1);
    int tn = t < taps ? next_tap(t) : taps;
    int chunk = 0, buf = 0;
    int32_t src_t[MT], src_tn[MT];
    u32x4 wreg[W_LOADS];
    u32x4 x_cur[KC / 16][MT], x_nxt[KC / 16][MT];
    load_src(t, src_t);
    load_src(tn, src_tn);
    if (t < taps) {
        fetch_w(t, 0, wreg);
        gather_x(src_t, 0, x_cur);
        store_w(0, wreg);
    }
    __syncthreads();
    while (t < taps) {
        const bool tap_ends = (chunk + 1 == chunks);
        const int t2 = tap_ends ? tn : t;
        const int chunk2 = tap_ends ? 0 : chunk + 1;
        const bool has_next = t2 < taps;
        int tnn = tn;
        int32_t src_tnn[MT];
#pragma unroll
        for (int a = 0; a < MT; ++a) src_tnn[a] = -1;
        if (has_next) {
            fetch_w(t2, chunk2 * KC, wreg);
            if (tap_ends) gather_x(src_tn, 0, x_nxt);
            else gather_x(src_t, chunk2 * KC, x_nxt);
            if (tap_ends) {
                tnn = next_tap(tn);
                load_src(tnn, src_tnn);
            }
        }
        bool wave_any = false;
#pragma unroll
        for (int a = 0; a < MT; ++a) wave_any |= (__ballot(src_t[a] >= 0) != 0);
        if (wave_any) {
#pragma unroll
            for (int ks = 0; ks < KC / 16; ++ks) {
                if (chunk * KC + ks * 16 < cin) {
#pragma unroll
                    for (int b = 0; b < NT; ++b) {
                        const v8 wfrag = __builtin_bit_cast(v8, *(const u32x4*)&w_lds[buf][b * 32 + col][ks * 16 + hf * 8]);
#pragma unroll
                        for (int a = 0; a < MT; ++a)
                            acc[a][b] = HalfOps<T>::mfma(wfrag, __builtin_bit_cast(v8, x_cur[ks][a]), acc[a][b]);
                    }
                }
            }
        }
        if (has_next) store_w(buf ^ 1, wreg);
        __syncthreads();
        buf ^= 1;
#pragma unroll
        for (int ks = 0; ks < KC / 16; ++ks)
#pragma unroll
            for (int a = 0; a < MT; ++a) x_cur[ks][a] = x_nxt[ks][a];
        if (tap_ends) {
#pragma unroll
            for (int a = 0; a < MT; ++a) { src_t[a] = src_tn[a]; src_tn[a] = src_tnn[a]; }
            t = tn;
            tn = tnn;
        }
        chunk = chunk2;
    }

    // acc[a][b][v]: output channel cout0 + b*32 + 8*(v/4) + 4*hf + v%4 of row[a]
#pragma unroll
    for (int a = 0; a < MT; ++a) {
        int64_t orow;
        if (PAIRS) {
            if (row[a] < 0) continue;
            orow = pair_slot[row[a]];
        } else {
            if (row[a] >= n) continue;
            orow = row[a];
        }
#pragma unroll
        for (int b = 0; b < NT; ++b) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int co = cout0 + b * 32 + 8 * g + 4 * hf;
                if (co >= cout) continue;
                float r[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    r[q] = acc[a][b][4 * g + q] + ((!PAIRS && bias) ? HalfOps<T>::to_float(bias[co + q]) : 0.f);
                u32x2 pk = {HalfOps<T>::pack2(r[0], r[1]), HalfOps<T>::pack2(r[2], r[3])};
                *(u32x2*)(out + orow * cout + co) = pk;
            }
        }
    }
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

template <typename T, int MT, int NT, int KC>
void launch_dense_kc(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps, bool tap_major,
                  const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    dim3 grid((unsigned)ptv3_ceil_div(n, ROWS), (unsigned)ptv3_ceil_div(cout, COUT_TILE));
    hipLaunchKernelGGL((subm_conv_gemm_kernel<T, MT, NT, KC, false>), grid, dim3(CONV_THREADS), 0, stream,
                       (const T*)feat, n, cin, nbr, taps, tap_major, (const T*)weight, (const T*)bias, cout, (T*)out,
                       (const int32_t*)nullptr, (const int32_t*)nullptr, (const int32_t*)nullptr);
}

template <typename T, int MT, int NT>
void launch_dense(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps, bool tap_major,
                  const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    // wide channel slices cut the number of barriers; thin inputs would only pad them with zeros
    if (cin >= 64) launch_dense_kc<T, MT, NT, 64>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
    else launch_dense_kc<T, MT, NT, 32>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
}

template <typename T>
void dispatch_dense(const void* feat, int64_t n, int cin, const int32_t* nbr, int taps, bool tap_major,
                    const void* weight, const void* bias, int cout, void* out, hipStream_t stream) {
    // Rows per work-group: 256 while that still yields >= ~2 work-groups per CU, else 128.
    const int64_t col_tiles = cout <= 32 ? 1 : (cout <= 64 ? 1 : ptv3_ceil_div(cout, 128));
    const bool wide = ptv3_ceil_div(n, 256) * col_tiles >= 512;
    if (cout <= 32) {
        if (wide) launch_dense<T, 2, 1>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
        else launch_dense<T, 1, 1>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
    } else if (cout <= 64) {
        if (wide) launch_dense<T, 2, 2>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
        else launch_dense<T, 1, 2>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
    } else {
        if (wide) launch_dense<T, 2, 4>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
        else launch_dense<T, 1, 4>(feat, n, cin, nbr, taps, tap_major, weight, bias, cout, out, stream);
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
    for (int s = s0; s < s1; ++s) {
        const v8 v = __builtin_bit_cast(v8, *(const u32x4*)(y + (int64_t)s * cout + c));
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[k] += (float)v[k];
    }
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = HalfOps<T>::pack2(acc[2 * k], acc[2 * k + 1]);
    *(u32x4*)(out + i * cout + c) = r;
}

template <typename T, int MT, int NT, int KC>
void launch_pairs_kc(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                     const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout,
                     void* y, hipStream_t stream) {
    constexpr int ROWS = CONV_WAVES * MT * 32, COUT_TILE = NT * 32;
    // every tap may end with one partial tile
    dim3 grid((unsigned)(n_pairs / ROWS + taps), (unsigned)ptv3_ceil_div(cout, COUT_TILE));
    hipLaunchKernelGGL((subm_conv_gemm_kernel<T, MT, NT, KC, true>), grid, dim3(CONV_THREADS), 0, stream,
                       (const T*)feat, (int64_t)0, cin, (const int32_t*)nullptr, taps, false, (const T*)weight,
                       (const T*)nullptr, cout, (T*)y, pair_in, pair_slot, tap_ptr);
}

template <typename T, int MT, int NT>
void launch_pairs(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                  const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                  hipStream_t stream) {
    if (cin >= 64)
        launch_pairs_kc<T, MT, NT, 64>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
    else
        launch_pairs_kc<T, MT, NT, 32>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
}

template <typename T>
void dispatch_pairs(const void* feat, int cin, int taps, int64_t n_pairs, const int32_t* tap_ptr,
                    const int32_t* pair_in, const int32_t* pair_slot, const void* weight, int cout, void* y,
                    hipStream_t stream) {
    const int64_t col_tiles = cout <= 64 ? 1 : ptv3_ceil_div(cout, 128);
    const bool wide = (n_pairs / 256 + taps) * col_tiles >= 512;
#define PTV3_PAIRS(MT, NT) launch_pairs<T, MT, NT>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream)
    if (cout <= 32) { if (wide) PTV3_PAIRS(2, 1); else PTV3_PAIRS(1, 1); }
    else if (cout <= 64) { if (wide) PTV3_PAIRS(2, 2); else PTV3_PAIRS(1, 2); }
    else { if (wide) PTV3_PAIRS(2, 4); else PTV3_PAIRS(1, 4); }
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
    if (cin % 16 != 0 || cout % 4 != 0) return PTV3_ESHAPE;
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
    if (dtype == PTV3_F16) {
        if (n_pairs > 0)
            dispatch_pairs<_Float16>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
        hipLaunchKernelGGL(pair_segment_sum_kernel<_Float16>, sgrid, sblock, 0, stream, (const _Float16*)y,
                           row_ptr, n, cout, (const _Float16*)bias, (_Float16*)out);
    } else {
        if (n_pairs > 0)
            dispatch_pairs<__bf16>(feat, cin, taps, n_pairs, tap_ptr, pair_in, pair_slot, weight, cout, y, stream);
        hipLaunchKernelGGL(pair_segment_sum_kernel<__bf16>, sgrid, sblock, 0, stream, (const __bf16*)y, row_ptr,
                           n, cout, (const __bf16*)bias, (__bf16*)out);
    }
    PTV3_RETURN_LAUNCH();
}
