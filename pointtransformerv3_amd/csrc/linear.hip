// Linear layer for many rows and few channels: out = act(x W^T + b), x (n, K) with K = 32, 64, 128,
// 256 or 512, W (N, K) as nn.Linear stores it, half precision.
//
// The Linear layers of the wide blocks (model.py:541-545 cpe.1, :450 qkv, :487 proj, :510-512
// fc1 + GELU) are tall and skinny: 9k-150k rows against 128-512 input channels. A library GEMM
// spends most of its time in the prologue and epilogue of its K loop there. Here the contraction
// has no loop over memory at all: a wave owns 32 rows, converts them once to MFMA operand
// registers (K / 16 fragments) and multiplies them with one 32-channel tile of W after the other,
// W's chunk of output channels sitting in LDS for the life of the persistent work-group
// (products are taken transposed, rows of the A operand = output channels, so a lane ends up with
// 4 consecutive output channels of one row). x is read once per chunk of output channels, out is
// written once; rows move between global memory and registers as contiguous 16-byte pieces
// through a wave-private LDS buffer. The bias, and for fc1 the exact GELU, are applied on the
// accumulators; results are rounded to the storage type once, as the separate layers round.
#include "rowtile.h"

namespace {

constexpr int LIN_PAD = 8;                 // halfs of padding per LDS row
// LDS budget for the weight chunk: at 128 inputs small enough for two work-groups per CU
constexpr size_t lin_w_bytes(int k) { return k <= 128 ? 40 * 1024 : 105 * 1024; }

// inference BatchNorm folded into the epilogue (model.py:726-735: Linear -> BatchNorm1d -> GELU)
struct LinBn {
    const void* mean;    // running statistics: float32 when stats_f32, else of the data type
    const void* var;
    const void* gamma;   // of the data type, or null
    const void* beta;
    float eps;
    int stats_f32;
};

// what follows the bias (and the BatchNorm): nothing, the exact GELU, the GELU with the value in front of it
// kept in aux as well (training: its backward needs it), or a multiplication by gelu'(aux) -- the input
// gradient of a Linear whose input came out of a GELU (model.py:505-507, fc2 back through act)
enum { ACT_NONE = 0, ACT_GELU = 1, ACT_GELU_KEEP = 2, ACT_GELU_GRAD = 3 };

// NW waves per work-group, rows staged SW channels at a time (64, or 32 where the weights leave LDS for
// narrow tile buffers only and the work-group has 16 waves instead of 8)
template <typename T, int K, int ACT, bool BN, int NW, int SW>
__global__ __launch_bounds__(NW * PTV3_WAVE, (NW == 8 ? 2 : 1)) void linear_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, LinBn bn, int64_t n, int nout,
    int chunk, int per_chunk, int n_chunks, T* __restrict__ out, T* __restrict__ aux) {
    typedef typename H16<T>::v8 v8;
    constexpr int KS = K / 16, WS = K + LIN_PAD, LIN_THREADS = NW * PTV3_WAVE, LIN_WAVES = NW, LIN_XSS = SW + LIN_PAD;
    extern __shared__ __align__(16) unsigned char lin_smem[];
    T* w_lds = (T*)lin_smem;                               // [chunk][WS]
    float* b_lds = (float*)(w_lds + (size_t)chunk * WS);   // [chunk]
    float* mu_lds = b_lds + chunk;                         // [chunk] x 3 with BN: mean, rstd * gamma, beta
    float* sc_lds = mu_lds + (BN ? chunk : 0);
    float* be_lds = sc_lds + (BN ? chunk : 0);
    T* xs_all = (T*)(be_lds + (BN ? chunk : 0));           // [waves][32][LIN_XSS]

    // Work-groups go to the 8 XCDs round-robin and every XCD has its own L2: the n_chunks work-groups that walk
    // the same rows (one per chunk of output channels) are dealt to one XCD, next to each other, so the rows
    // leave HBM once. The walks themselves stay interleaved over the XCDs in launch order (with one chunk this
    // is the plain order; handing each XCD a contiguous eighth of the rows measured 5-20 % slower).
    // per_chunk < 0: the walks do not spread evenly over 8 XCDs that way; chunk-major launch order instead.
    int row_group, chunk_id;
    if (per_chunk > 0) {
        const int slot = blockIdx.x >> 3;
        row_group = (slot / n_chunks) * 8 + (blockIdx.x & 7);   // which of the per_chunk walks over the row tiles
        chunk_id = slot % n_chunks;
    } else {
        per_chunk = -per_chunk;
        row_group = blockIdx.x % per_chunk;
        chunk_id = blockIdx.x / per_chunk;
    }
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    T* xs = xs_all + wave * (32 * LIN_XSS);
    const int c0 = chunk_id * chunk;                       // first output channel of this work-group
    const int cn = min(chunk, nout - c0);                  // its output channels (a multiple of 32)

    // ---- weight chunk and bias -> LDS (rows past cn are never read)
    {
        constexpr int PPR = K / 8;
        for (int e = tid; e < cn * PPR; e += LIN_THREADS) {
            const int r = e / PPR, pc = e % PPR;
            *(u32x4*)(w_lds + r * WS + pc * 8) = *(const u32x4*)(w + (int64_t)(c0 + r) * K + pc * 8);
        }
        for (int e = tid; e < cn; e += LIN_THREADS) {
            b_lds[e] = bias ? (float)bias[c0 + e] : 0.f;
            if (BN) {
                const int c = c0 + e;
                const float mu = bn.stats_f32 ? ((const float*)bn.mean)[c] : (float)((const T*)bn.mean)[c];
                const float va = bn.stats_f32 ? ((const float*)bn.var)[c] : (float)((const T*)bn.var)[c];
                mu_lds[e] = mu;
                sc_lds[e] = rsqrtf(va + bn.eps) * (bn.gamma ? (float)((const T*)bn.gamma)[c] : 1.f);
                be_lds[e] = bn.beta ? (float)((const T*)bn.beta)[c] : 0.f;
            }
        }
    }
    __syncthreads();

    const int64_t n_tiles = (n + 31) / 32;
    constexpr int PART = K < SW ? K : SW;             // channels staged at a time
    constexpr int PPP = PART / 8;                     // 16-byte pieces per row and part
    constexpr int ITS = 32 * PPP / PTV3_WAVE;         // pieces per lane and part
    constexpr int PARTS = K / PART;
    // Up to 128 inputs a wave's 32 rows are 32 registers per lane: the next tile's rows are requested before this
    // tile's products start, so their way from HBM is covered by a whole tile of work instead of by the other
    // waves of the SIMD alone: 2-5 % on the plain layers. (At 256 and 512 inputs the operand fragments leave no
    // room for a second set, and with the BatchNorm / GELU epilogues the extra registers cost a wave per SIMD.)
    constexpr bool AHEAD = K <= 128 && !BN && ACT == ACT_NONE;
    auto fetch = [&](int64_t t, u32x4 (&raw)[PARTS][ITS]) {
        const int64_t r0 = t * 32;
#pragma unroll
        for (int part = 0; part < PARTS; ++part)
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int pidx = it * PTV3_WAVE + lane;    // 32 rows x PPP pieces
                const int64_t r = r0 + pidx / PPP;
                raw[part][it] = (u32x4){0, 0, 0, 0};
                if (r < n) raw[part][it] = *(const u32x4*)(x + r * K + part * PART + (pidx % PPP) * 8);
            }
    };
    const int64_t stride = (int64_t)per_chunk * LIN_WAVES;
    u32x4 ahead[AHEAD ? PARTS : 1][AHEAD ? ITS : 1];
    int64_t tile = (int64_t)row_group * LIN_WAVES + wave;
    if constexpr (AHEAD) {
        if (tile < n_tiles) fetch(tile, ahead);
    }
    for (; tile < n_tiles; tile += stride) {
        const int64_t row0 = tile * 32;
        // ---- 32 rows -> operand fragments, 64 channels at a time: lane (r, piece) moves 16 bytes
        v8 xf[KS];
        u32x4 raw[PARTS][ITS];
        if constexpr (AHEAD) {
#pragma unroll
            for (int part = 0; part < PARTS; ++part)
#pragma unroll
                for (int it = 0; it < ITS; ++it) raw[part][it] = ahead[part][it];
            if (tile + stride < n_tiles) fetch(tile + stride, ahead);
        } else {
            fetch(tile, raw);
        }
#pragma unroll
        for (int part = 0; part < PARTS; ++part) {
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int pidx = it * PTV3_WAVE + lane;
                *(u32x4*)(xs + (pidx / PPP) * LIN_XSS + (pidx % PPP) * 8) = raw[part][it];
            }
            asm volatile("" ::: "memory");
#pragma unroll
            for (int ks = 0; ks < PART / 16; ++ks)
                xf[part * (PART / 16) + ks] = __builtin_bit_cast(v8, *(const u32x4*)(xs + col * LIN_XSS + ks * 16 + hf * 8));
            asm volatile("" ::: "memory");
        }
        // ---- output channels SW at a time (two 32-tiles, or one)
        for (int o0 = 0; o0 < cn; o0 += SW) {
            const int nt = (cn - o0) >= SW ? SW / 32 : 1;
            const int ppr_g = nt * 4;                        // 16-byte pieces per row of this group
            const int its = 32 * ppr_g / PTV3_WAVE;          // 4 or 2
            u32x4 pre[ACT == ACT_GELU_GRAD ? 4 : 1];         // the GELU's inputs at the places this lane writes
            if (ACT == ACT_GELU_GRAD) {
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    if (it >= its) break;
                    const int pidx = it * PTV3_WAVE + lane;
                    const int64_t r = row0 + pidx / ppr_g;
                    pre[it] = (u32x4){0, 0, 0, 0};
                    if (r < n) pre[it] = *(const u32x4*)(aux + r * nout + c0 + o0 + (pidx % ppr_g) * 8);
                }
            }
            u32x2 act[ACT == ACT_GELU_KEEP ? SW / 32 : 1][4];   // the activated values while the plain ones go out
#pragma unroll
            for (int t = 0; t < SW / 32; ++t) {
                if (t >= nt) break;
                f32x16 d;
#pragma unroll
                for (int v = 0; v < 16; ++v) d[v] = 0.f;
                const T* wrow = w_lds + (o0 + t * 32 + col) * WS + hf * 8;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(wrow + ks * 16)), xf[ks], d);
                // d[v]: output channel o0 + 32 t + 8 (v / 4) + 4 hf + v % 4 of row `col`
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 bb = *(const f32x4*)(b_lds + o0 + t * 32 + 8 * g + 4 * hf);
                    float r[4], a[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        r[q] = d[4 * g + q] + bb[q];
                        if (BN) {
                            const int c = o0 + t * 32 + 8 * g + 4 * hf + q;
                            r[q] = (H16<T>::round(r[q]) - mu_lds[c]) * sc_lds[c] + be_lds[c];
                        }
                        if (ACT == ACT_GELU) r[q] = gelu_erf(H16<T>::round(r[q]));
                        if (ACT == ACT_GELU_KEEP) a[q] = gelu_erf(H16<T>::round(r[q]));
                    }
                    *(u32x2*)(xs + col * LIN_XSS + t * 32 + 8 * g + 4 * hf) =
                        (u32x2){H16<T>::pack2(r[0], r[1]), H16<T>::pack2(r[2], r[3])};
                    if (ACT == ACT_GELU_KEEP) act[t][g] = (u32x2){H16<T>::pack2(a[0], a[1]), H16<T>::pack2(a[2], a[3])};
                }
            }
            asm volatile("" ::: "memory");
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                if (it >= its) break;
                const int pidx = it * PTV3_WAVE + lane;
                const int rr = pidx / ppr_g, pc = pidx % ppr_g;
                const int64_t r = row0 + rr;
                u32x4 o4 = *(const u32x4*)(xs + rr * LIN_XSS + pc * 8);
                if (ACT == ACT_GELU_GRAD) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t hw = pre[it][q], dw = o4[q];
                        o4[q] = H16<T>::pack2(H16<T>::lo(dw) * gelu_erf_grad(H16<T>::lo(hw)),
                                              H16<T>::hi(dw) * gelu_erf_grad(H16<T>::hi(hw)));
                    }
                }
                if (r < n) *(u32x4*)((ACT == ACT_GELU_KEEP ? aux : out) + r * nout + c0 + o0 + pc * 8) = o4;
            }
            asm volatile("" ::: "memory");
            if (ACT == ACT_GELU_KEEP) {
#pragma unroll
                for (int t = 0; t < SW / 32; ++t) {
                    if (t >= nt) break;
#pragma unroll
                    for (int g = 0; g < 4; ++g) *(u32x2*)(xs + col * LIN_XSS + t * 32 + 8 * g + 4 * hf) = act[t][g];
                }
                asm volatile("" ::: "memory");
#pragma unroll
                for (int it = 0; it < 4; ++it) {
                    if (it >= its) break;
                    const int pidx = it * PTV3_WAVE + lane;
                    const int rr = pidx / ppr_g, pc = pidx % ppr_g;
                    const int64_t r = row0 + rr;
                    const u32x4 o4 = *(const u32x4*)(xs + rr * LIN_XSS + pc * 8);
                    if (r < n) *(u32x4*)(out + r * nout + c0 + o0 + pc * 8) = o4;
                }
                asm volatile("" ::: "memory");
            }
        }
    }
}

template <typename T, int K, int ACT, bool BN, int NW, int SW>
int launch_linear_shape(const void* x, const void* w, const void* bias, LinBn bn, int64_t n, int nout, void* out,
                        void* aux, hipStream_t stream) {
    // output channels per work-group: as many 32-tiles as the LDS budget holds, spread evenly
    const int cap = (int)(lin_w_bytes(K) / ((K + LIN_PAD) * sizeof(T))) / 32 * 32;
    const int n_chunks = (nout + cap - 1) / cap;
    const int chunk = ((nout + n_chunks - 1) / n_chunks + 31) / 32 * 32;
    constexpr int LIN_WAVES = NW, LIN_THREADS = NW * PTV3_WAVE, LIN_XSS = SW + LIN_PAD;
    const size_t lds = (size_t)chunk * (K + LIN_PAD) * sizeof(T) + (size_t)chunk * sizeof(float) * (BN ? 4 : 1) +
                       (size_t)LIN_WAVES * 32 * LIN_XSS * sizeof(T);
    auto kern = linear_rows_kernel<T, K, ACT, BN, NW, SW>;
    static LdsGrant grant_lds_allowed;   // per instantiation and device; raised monotonically
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_lds_allowed)) return rc_;
    // persistent work-groups: as many as the LDS lets a CU hold, shared out between the chunks
    const int64_t tiles = (n + 31) / 32;
    int64_t per_chunk = ((lds <= 80 * 1024 && NW == 8) ? 512 : 256) / n_chunks;
    if (per_chunk < 1) per_chunk = 1;
    const int64_t need = (tiles + LIN_WAVES - 1) / LIN_WAVES;
    if (per_chunk > need) per_chunk = need;
    // several chunks and a number of walks that spreads evenly over the XCDs: chunks of a walk on one XCD (see
    // the kernel); cutting the walks down to a multiple of 8 for the other shapes measured slower than it gained
    const bool by_xcd = n_chunks > 1 && per_chunk % 8 == 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)(per_chunk * n_chunks)), dim3(LIN_THREADS), lds, stream, (const T*)x,
                       (const T*)w, (const T*)bias, bn, n, nout, chunk, (int)(by_xcd ? per_chunk : -per_chunk), n_chunks,
                       (T*)out, (T*)aux);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

template <typename T, int K, int ACT, bool BN>
int launch_linear(const void* x, const void* w, const void* bias, LinBn bn, int64_t n, int nout, void* out, void* aux,
                  hipStream_t stream) {
    // 256 inputs with GELU: the weight chunk takes the LDS of the whole CU and the epilogue is VALU-heavy, so one
    // work-group of 16 waves with 32-channel tile buffers (four waves per SIMD) measured 13 % faster than 8 waves;
    // without GELU, and at 512 inputs where the x fragments alone need 128 registers, the 8-wave shape is faster
    if constexpr (K == 256 && ACT != ACT_NONE)
        return launch_linear_shape<T, K, ACT, BN, 16, 32>(x, w, bias, bn, n, nout, out, aux, stream);
    return launch_linear_shape<T, K, ACT, BN, 8, 64>(x, w, bias, bn, n, nout, out, aux, stream);
}

// act: one of ACT_*; the BatchNorm epilogue comes with ACT_NONE and ACT_GELU only
int dispatch_linear(const void* x, const void* w, const void* bias, const LinBn* bn, int dtype, int64_t n, int k,
                    int nout, int act, void* out, void* aux, hipStream_t stream) {
    const LinBn none = {nullptr, nullptr, nullptr, nullptr, 0.f, 0};
#define PTV3_LIN(T, K)                                                                                                \
    if (k == K) {                                                                                                     \
        if (bn) return act ? launch_linear<T, K, ACT_GELU, true>(x, w, bias, *bn, n, nout, out, aux, stream)          \
                           : launch_linear<T, K, ACT_NONE, true>(x, w, bias, *bn, n, nout, out, aux, stream);         \
        switch (act) {                                                                                                \
            case ACT_NONE: return launch_linear<T, K, ACT_NONE, false>(x, w, bias, none, n, nout, out, aux, stream);  \
            case ACT_GELU: return launch_linear<T, K, ACT_GELU, false>(x, w, bias, none, n, nout, out, aux, stream);  \
            case ACT_GELU_KEEP:                                                                                       \
                return launch_linear<T, K, ACT_GELU_KEEP, false>(x, w, bias, none, n, nout, out, aux, stream);        \
            default: return launch_linear<T, K, ACT_GELU_GRAD, false>(x, w, bias, none, n, nout, out, aux, stream);   \
        }                                                                                                             \
    }
    if (dtype == PTV3_F16) {
        PTV3_LIN(_Float16, 32) PTV3_LIN(_Float16, 64) PTV3_LIN(_Float16, 128) PTV3_LIN(_Float16, 256) PTV3_LIN(_Float16, 512)
    } else {
        PTV3_LIN(__bf16, 32) PTV3_LIN(__bf16, 64) PTV3_LIN(__bf16, 128) PTV3_LIN(__bf16, 256) PTV3_LIN(__bf16, 512)
    }
#undef PTV3_LIN
    return PTV3_ESHAPE;
}

// The general shape: any number of inputs and outputs, fp32 as well as fp16 / bf16, plain FMA arithmetic in
// fp32 on 64 x 64 output tiles with 16-input slices of x and w in LDS. It serves the fp32 model (the
// reference's parity path, model.py:458-474 with enable_flash=False) and half-precision layers whose widths the
// MFMA kernels above do not take; not tuned.
constexpr int ANY_TILE = 64, ANY_KC = 16;

template <typename T> __device__ __forceinline__ float any_f(T v) { return (float)v; }

template <typename T>
__global__ __launch_bounds__(256) void linear_any_kernel(const T* x, const T* w, const T* bias, const T* resid,
                                                         int64_t n, int k, int nout, int gelu, T* out) {
    __shared__ float xs[ANY_KC][ANY_TILE + 1];
    __shared__ float ws[ANY_KC][ANY_TILE + 1];
    const int tid = threadIdx.x, tr = tid / 16, tc = tid % 16;
    const int64_t row0 = (int64_t)blockIdx.x * ANY_TILE;
    const int col0 = blockIdx.y * ANY_TILE;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < k; k0 += ANY_KC) {
#pragma unroll
        for (int e = tid; e < ANY_TILE * ANY_KC; e += 256) {
            const int r = e / ANY_KC, kk = e % ANY_KC;
            const bool in_k = k0 + kk < k;
            xs[kk][r] = (in_k && row0 + r < n) ? any_f(x[(row0 + r) * k + k0 + kk]) : 0.f;
            ws[kk][r] = (in_k && col0 + r < nout) ? any_f(w[(int64_t)(col0 + r) * k + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < ANY_KC; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][tr + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tc + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t r = row0 + tr + 16 * i;
            const int c = col0 + tc + 16 * j;
            if (r >= n || c >= nout) continue;
            float v = acc[i][j] + (bias ? any_f(bias[c]) : 0.f);
            if (gelu) v = 0.5f * v * (1.f + erff(v * 0.70710678118654752f));
            if (resid) v += any_f(resid[r * nout + c]);
            out[r * nout + c] = (T)v;
        }
}

template <typename T>
int launch_linear_any(const void* x, const void* w, const void* bias, const void* resid, int64_t n, int k, int nout,
                      int gelu, void* out, hipStream_t stream) {
    const dim3 grid((unsigned)ptv3_ceil_div(n, ANY_TILE), (unsigned)ptv3_ceil_div(nout, ANY_TILE));
    hipLaunchKernelGGL(linear_any_kernel<T>, grid, dim3(256), 0, stream, (const T*)x, (const T*)w, (const T*)bias,
                       (const T*)resid, n, k, nout, gelu, (T*)out);
    PTV3_RETURN_LAUNCH();
}

int check_linear(int dtype, int64_t n, int k, int nout) {
    if (n < 0 || k < 1 || nout < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if ((k != 32 && k != 64 && k != 128 && k != 256 && k != 512) || nout % 32 != 0) return PTV3_ESHAPE;
    return PTV3_OK;
}

}  // namespace

extern "C" int ptv3_linear_fwd(const void* x, const void* w, const void* bias, int dtype, int64_t n, int k, int nout,
                               int gelu, void* out, void* stream_) {
    const int rc = check_linear(dtype, n, k, nout);
    if (rc != PTV3_OK) return rc;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !out) return PTV3_EINVAL;
    return dispatch_linear(x, w, bias, nullptr, dtype, n, k, nout, gelu ? ACT_GELU : ACT_NONE, out, nullptr,
                           (hipStream_t)stream_);
}

extern "C" int ptv3_linear_gelu_fwd(const void* x, const void* w, const void* bias, int dtype, int64_t n, int k,
                                    int nout, void* pre, void* out, void* stream_) {
    const int rc = check_linear(dtype, n, k, nout);
    if (rc != PTV3_OK) return rc;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !pre || !out) return PTV3_EINVAL;
    return dispatch_linear(x, w, bias, nullptr, dtype, n, k, nout, ACT_GELU_KEEP, out, pre, (hipStream_t)stream_);
}

extern "C" int ptv3_linear_gelu_bwd(const void* dout, const void* wt, const void* pre, int dtype, int64_t n, int k,
                                    int nout, void* dpre, void* stream_) {
    const int rc = check_linear(dtype, n, k, nout);
    if (rc != PTV3_OK) return rc;
    if (n == 0) return PTV3_OK;
    if (!dout || !wt || !pre || !dpre) return PTV3_EINVAL;
    return dispatch_linear(dout, wt, nullptr, nullptr, dtype, n, k, nout, ACT_GELU_GRAD, dpre, const_cast<void*>(pre),
                           (hipStream_t)stream_);
}

extern "C" int ptv3_linear_bn_act_fwd(const void* x, const void* w, const void* bias, const void* running_mean,
                                      const void* running_var, int stats_f32, const void* gamma, const void* beta,
                                      float eps, int dtype, int64_t n, int k, int nout, int gelu, void* out,
                                      void* stream_) {
    const int rc = check_linear(dtype, n, k, nout);
    if (rc != PTV3_OK) return rc;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !running_mean || !running_var || !out) return PTV3_EINVAL;
    const LinBn bn = {running_mean, running_var, gamma, beta, eps, stats_f32};
    return dispatch_linear(x, w, bias, &bn, dtype, n, k, nout, gelu ? ACT_GELU : ACT_NONE, out, nullptr,
                           (hipStream_t)stream_);
}

extern "C" int ptv3_linear_any_fwd(const void* x, const void* w, const void* bias, const void* resid, int dtype,
                                   int64_t n, int k, int nout, int gelu, void* out, void* stream_) {
    if (n < 0 || k < 1 || nout < 1 || ptv3_ceil_div(n, ANY_TILE) >= (1ll << 31)) return PTV3_EINVAL;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    switch (dtype) {
        case PTV3_F32: return launch_linear_any<float>(x, w, bias, resid, n, k, nout, gelu, out, stream);
        case PTV3_F16: return launch_linear_any<_Float16>(x, w, bias, resid, n, k, nout, gelu, out, stream);
        case PTV3_BF16: return launch_linear_any<__bf16>(x, w, bias, resid, n, k, nout, gelu, out, stream);
        default: return PTV3_EINVAL;
    }
}
