// Square Linear layer with the LayerNorms and residual additions that follow it in a wide PTv3 block,
// in one kernel: the row never leaves the registers between the GEMM and the normalisation.
//
//   mode 2 (after attention, model.py:594-597): s = res + Linear(x); out0 = s (+ shift); out1 = LN(s)
//          (proj, then the residual and the MLP's pre-norm; `shift` is the bias of the GEMM that will
//          accumulate onto out0 later, as in the LayerNorm kernel's mode 2)
//   mode 3 (xCPE, model.py:587-593): s = res + LN(Linear(x)); out0 = s; out1 = LN2(s)
//          (cpe.1 Linear, cpe.2 LayerNorm, the residual, then the attention's pre-norm)
// for C = 128 channels in and out (64 and below are covered by the block head / tail kernels; 256 by the
// kernel that keeps the weights in registers, linear_wide_kernel with its LN modes). Every intermediate is rounded to the storage type exactly where the separate kernels
// store it (Linear output, normalised value, sum), so fusing changes no value.
//
// Structure as the tall-and-skinny Linear kernel: a wave owns 32 rows as K/16 MFMA operand fragments,
// all C x C weights sit in LDS for the life of the persistent work-group, products are transposed
// (a lane ends up with 4 consecutive output channels of one row, 8 times per 32-channel tile). Here
// all C/32 accumulator tiles stay live, so lane (row, half) holds half of its row and a row's
// statistics are a sum over registers plus one exchange with lane ^ 32. Rows move between global
// memory and registers as contiguous 16-byte pieces through a wave-private LDS buffer, 64 channels
// at a time.
#include "rowtile.h"

namespace {

constexpr int LL_PAD = 8;              // halfs of padding per LDS weight row
constexpr int LL_XSS = 64 + LL_PAD;    // tile buffer row stride: 64 channels at a time

template <int C> struct LlShape {
    static constexpr int WAVES = 8;
    static constexpr int THREADS = WAVES * PTV3_WAVE;
    static constexpr int OCC = 1;                      // a row's C outputs stay in registers: 256 per lane
    static constexpr size_t LDS = (size_t)C * (C + LL_PAD) * 2 + (size_t)6 * C * 4 + (size_t)WAVES * 32 * LL_XSS * 2;
};

template <typename T, int C, int MODE>
__global__ __launch_bounds__(LlShape<C>::THREADS, LlShape<C>::OCC) void linear_ln_kernel(
    const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias, const T* __restrict__ res,
    const T* __restrict__ gamma, const T* __restrict__ beta, const T* __restrict__ gamma2,
    const T* __restrict__ beta2, const T* __restrict__ shift, int64_t n, float eps, T* __restrict__ out0,
    T* __restrict__ out1) {
    typedef typename H16<T>::v8 v8;
    constexpr int KS = C / 16, WS = C + LL_PAD, NT = C / 32, THREADS = LlShape<C>::THREADS, WAVES = LlShape<C>::WAVES;
    extern __shared__ __align__(16) unsigned char ll_smem[];
    T* w_lds = (T*)ll_smem;                            // [C][WS]
    float* p_lds = (float*)(w_lds + (size_t)C * WS);   // [6][C]: bias, gamma, beta, gamma2, beta2, shift
    T* xs_all = (T*)(p_lds + 6 * C);                   // [waves][32][LL_XSS]

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    T* xs = xs_all + wave * (32 * LL_XSS);

    {
        constexpr int PPR = C / 8;
        for (int e = tid; e < C * PPR; e += THREADS) {
            const int r = e / PPR, pc = e % PPR;
            *(u32x4*)(w_lds + r * WS + pc * 8) = *(const u32x4*)(w + (int64_t)r * C + pc * 8);
        }
        for (int e = tid; e < C; e += THREADS) {
            p_lds[e] = bias ? (float)bias[e] : 0.f;
            p_lds[C + e] = (float)gamma[e];
            p_lds[2 * C + e] = (float)beta[e];
            p_lds[3 * C + e] = MODE == 3 ? (float)gamma2[e] : 0.f;
            p_lds[4 * C + e] = MODE == 3 ? (float)beta2[e] : 0.f;
            p_lds[5 * C + e] = (MODE == 2 && shift) ? (float)shift[e] : 0.f;
        }
    }
    __syncthreads();

    // 32 rows x 64 channels between global memory (row stride C) and the wave's tile buffer
    constexpr int ITS = 32 * 8 / PTV3_WAVE;   // 16-byte pieces per lane
    auto slab_in = [&](const T* src, int64_t row0, int ch0) {
        u32x4 raw[ITS];
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / 8;
            raw[it] = (u32x4){0, 0, 0, 0};
            if (r < n) raw[it] = *(const u32x4*)(src + r * C + ch0 + (pidx % 8) * 8);
        }
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            *(u32x4*)(xs + (pidx / 8) * LL_XSS + (pidx % 8) * 8) = raw[it];
        }
        asm volatile("" ::: "memory");
    };
    auto slab_out = [&](T* dst, int64_t row0, int ch0) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / 8;
            const u32x4 o4 = *(const u32x4*)(xs + (pidx / 8) * LL_XSS + (pidx % 8) * 8);
            if (r < n) *(u32x4*)(dst + r * C + ch0 + (pidx % 8) * 8) = o4;
        }
        asm volatile("" ::: "memory");
    };
    // channel of accumulator element v of tile t in this lane: 32 t + 8 (v / 4) + 4 hf + v % 4
    auto stats = [&](const float (&val)[NT][16], float& mean, float& rstd) {
        float s = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) s += val[t][v];
        s += __shfl_xor(s, 32, PTV3_WAVE);
        mean = s * (1.f / C);
        float q = 0.f;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) q += (val[t][v] - mean) * (val[t][v] - mean);
        q += __shfl_xor(q, 32, PTV3_WAVE);
        rstd = rsqrtf(q * (1.f / C) + eps);
    };
    // this lane's pieces of the staged slab <-> tiles 2 sl, 2 sl + 1
    auto put_slab = [&](const float (&val)[NT][16], int sl, const float* add) {
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int t = 2 * sl + tt, c = 32 * t + 8 * g + 4 * hf;
                float o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) o[q] = val[t][4 * g + q] + (add ? add[c + q] : 0.f);
                *(u32x2*)(xs + col * LL_XSS + tt * 32 + 8 * g + 4 * hf) =
                    (u32x2){H16<T>::pack2(o[0], o[1]), H16<T>::pack2(o[2], o[3])};
            }
    };

    const int64_t n_tiles = (n + 31) / 32;
    for (int64_t tile = (int64_t)blockIdx.x * WAVES + wave; tile < n_tiles; tile += (int64_t)gridDim.x * WAVES) {
        const int64_t row0 = tile * 32;
        // ---- rows -> operand fragments
        v8 xf[KS];
#pragma unroll
        for (int part = 0; part < C / 64; ++part) {
            slab_in(x, row0, part * 64);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
                xf[part * 4 + ks] = __builtin_bit_cast(v8, *(const u32x4*)(xs + col * LL_XSS + ks * 16 + hf * 8));
            asm volatile("" ::: "memory");
        }
        // ---- Linear: all C / 32 output tiles, rounded to the storage type with the bias
        float val[NT][16];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            f32x16 d;
#pragma unroll
            for (int v = 0; v < 16; ++v) d[v] = 0.f;
            const T* wrow = w_lds + (t * 32 + col) * WS + hf * 8;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(wrow + ks * 16)), xf[ks], d);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(p_lds + 32 * t + 8 * g + 4 * hf);
#pragma unroll
                for (int q = 0; q < 4; ++q) val[t][4 * g + q] = H16<T>::round(d[4 * g + q] + bb[q]);
            }
        }
        // ---- the residual rows, as packed halfs (this lane's pieces)
        uint32_t rp[NT][8];
#pragma unroll
        for (int sl = 0; sl < NT / 2; ++sl) {
            slab_in(res, row0, sl * 64);
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const u32x2 p = *(const u32x2*)(xs + col * LL_XSS + tt * 32 + 8 * g + 4 * hf);
                    rp[2 * sl + tt][2 * g] = p[0];
                    rp[2 * sl + tt][2 * g + 1] = p[1];
                }
            asm volatile("" ::: "memory");
        }
        float mean, rstd;
        if (MODE == 3) {
            // s = res + LN(lin), every stage rounded
            stats(val, mean, rstd);
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int c = 32 * t + 8 * g + 4 * hf;
                    const f32x4 ga = *(const f32x4*)(p_lds + C + c), be = *(const f32x4*)(p_lds + 2 * C + c);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t pw = rp[t][2 * g + q / 2];
                        const float r = (q & 1) ? H16<T>::hi(pw) : H16<T>::lo(pw);
                        const float y = (val[t][4 * g + q] - mean) * rstd * ga[q] + be[q];
                        val[t][4 * g + q] = H16<T>::round(H16<T>::round(y) + r);
                    }
                }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t pw = rp[t][2 * g + q / 2];
                        const float r = (q & 1) ? H16<T>::hi(pw) : H16<T>::lo(pw);
                        val[t][4 * g + q] = H16<T>::round(val[t][4 * g + q] + r);
                    }
        }
        // ---- out0 = s (+ shift), out1 = LN(s) with the second (mode 3) or only (mode 2) parameters
#pragma unroll
        for (int sl = 0; sl < NT / 2; ++sl) {
            put_slab(val, sl, MODE == 2 ? p_lds + 5 * C : nullptr);
            slab_out(out0, row0, sl * 64);
        }
        stats(val, mean, rstd);
        const float* ga_l = p_lds + (MODE == 3 ? 3 * C : C);
        const float* be_l = p_lds + (MODE == 3 ? 4 * C : 2 * C);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int c = 32 * t + 8 * g + 4 * hf;
                const f32x4 ga = *(const f32x4*)(ga_l + c), be = *(const f32x4*)(be_l + c);
#pragma unroll
                for (int q = 0; q < 4; ++q) val[t][4 * g + q] = (val[t][4 * g + q] - mean) * rstd * ga[q] + be[q];
            }
#pragma unroll
        for (int sl = 0; sl < NT / 2; ++sl) {
            put_slab(val, sl, nullptr);
            slab_out(out1, row0, sl * 64);
        }
    }
}

template <typename T, int C, int MODE>
int launch_linear_ln(const void* x, const void* w, const void* bias, const void* res, const void* gamma,
                     const void* beta, const void* gamma2, const void* beta2, const void* shift, int64_t n, float eps,
                     void* out0, void* out1, hipStream_t stream) {
    typedef LlShape<C> S;
    auto kern = linear_ln_kernel<T, C, MODE>;
    static LdsGrant grant_attr_set;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, S::LDS, grant_attr_set)) return rc_;
    const int64_t tiles = (n + 31) / 32;
    int64_t grid = 256 * S::OCC;
    const int64_t need = (tiles + S::WAVES - 1) / S::WAVES;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(S::THREADS), S::LDS, stream, (const T*)x, (const T*)w,
                       (const T*)bias, (const T*)res, (const T*)gamma, (const T*)beta, (const T*)gamma2, (const T*)beta2,
                       (const T*)shift, n, eps, (T*)out0, (T*)out1);
    PTV3_RETURN_LAUNCH();
}

template <typename T>
int dispatch_linear_ln(const void* x, const void* w, const void* bias, const void* res, const void* gamma,
                       const void* beta, const void* gamma2, const void* beta2, const void* shift, int64_t n, int c,
                       int mode, float eps, void* out0, void* out1, hipStream_t stream) {
#define PTV3_LL(C, M)                                                                                           \
    if (c == C && mode == M)                                                                                    \
        return launch_linear_ln<T, C, M>(x, w, bias, res, gamma, beta, gamma2, beta2, shift, n, eps, out0, out1, stream);
    PTV3_LL(128, 2) PTV3_LL(128, 3)
#undef PTV3_LL
    return PTV3_ESHAPE;
}

}  // namespace

int linear_wide_ln_dispatch(const void* x, const void* w, const void* bias, const void* res, const void* gamma,
                            const void* beta, const void* gamma2, const void* beta2, const void* shift, int dtype,
                            int64_t n, int mode, float eps, void* out0, void* out1, hipStream_t stream);

extern "C" int ptv3_linear_ln_fwd(const void* x, const void* w, const void* bias, const void* res, const void* gamma,
                                  const void* beta, const void* gamma2, const void* beta2, const void* shift, int dtype,
                                  int64_t n, int channels, int mode, float eps, void* out0, void* out1, void* stream_) {
    if (n < 0) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if ((channels != 128 && channels != 256) || (mode != 2 && mode != 3)) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !res || !gamma || !beta || !out0 || !out1) return PTV3_EINVAL;
    if (mode == 3 && (!gamma2 || !beta2)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    // 256 channels: the kernel that keeps the weights in registers (linearw.hip); below that they fit the LDS
    if (channels == 256)
        return linear_wide_ln_dispatch(x, w, bias, res, gamma, beta, gamma2, beta2, shift, dtype, n, mode, eps, out0, out1,
                                       stream);
    if (dtype == PTV3_F16)
        return dispatch_linear_ln<_Float16>(x, w, bias, res, gamma, beta, gamma2, beta2, shift, n, channels, mode, eps,
                                            out0, out1, stream);
    return dispatch_linear_ln<__bf16>(x, w, bias, res, gamma, beta, gamma2, beta2, shift, n, channels, mode, eps, out0,
                                      out1, stream);
}
