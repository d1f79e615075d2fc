// Fused transformer MLP for thin channels: out = resid + fc2(GELU(fc1(x))) in one kernel.
//
// Replaces, for C = 32 or 64 and hidden = 4C, the chain model.py:510-516 (fc1, GELU, fc2) plus the
// residual add of model.py:602. At these widths the layer is bound by the 4C-wide hidden tensor
// going to HBM and back four times (fc1 out, GELU in/out, fc2 in); here it never leaves the CU.
//
// Both weight matrices stay in LDS for the life of a (persistent) work-group; a wave takes 32 rows
// at a time. The products are taken transposed with v_mfma_f32_32x32x16:
//   H^T (32 hidden x 32 rows) = W1 (rows: hidden units) * X^T      -> each lane owns ONE input row
//   Out^T (C x 32 rows)      += W2 (rows: out channels) * GELU(H^T)
// so the fp32 results of the first product, after bias, rounding and GELU, are -- converted to
// 16 bit -- already the B operand of the second; W2's hidden axis is stored in the matching
// register order. Row tiles move between global memory and registers as contiguous 16-byte
// pieces through a wave-private LDS buffer.
// GELU is the exact erf form of nn.GELU (gelu_erf in rowtile.h: a one-ulp-level fit for half-precision results).
#include "rowtile.h"

namespace {

constexpr int MLP_THREADS = 512;
constexpr int MLP_WAVES = MLP_THREADS / PTV3_WAVE;
constexpr int PADH = 8;   // halfs of padding per LDS row

template <typename T, int C>
__global__ __launch_bounds__(MLP_THREADS, 2) void mlp_fused_kernel(
    const T* __restrict__ x, const T* __restrict__ resid, const T* __restrict__ w1,
    const T* __restrict__ b1, const T* __restrict__ w2, const T* __restrict__ b2, int64_t n,
    T* __restrict__ out) {
    typedef typename H16<T>::v8 v8;
    constexpr int H = 4 * C;
    constexpr int KS = C / 16;        // 16-channel steps of the first product
    constexpr int OT = C / 32;        // 32-channel tiles of the output
    constexpr int W1S = C + PADH;     // LDS row strides (halfs)
    constexpr int W2S = H + PADH;
    constexpr int XSS = C + PADH;
    extern __shared__ __align__(16) unsigned char mlp_smem[];
    T* w1_lds = (T*)mlp_smem;                      // [H][W1S]
    T* w2_lds = w1_lds + H * W1S;                  // [C][W2S], hidden axis permuted per 32-block
    float* b1_lds = (float*)(w2_lds + C * W2S);    // [H]
    float* b2_lds = b1_lds + H;                    // [C]
    T* xs_all = (T*)(b2_lds + C);                  // [waves][32][XSS]

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    T* xs = xs_all + wave * (32 * XSS);

    // ---- weights and biases into LDS, once
    for (int e = tid; e < H * (C / 8); e += MLP_THREADS) {
        const int r = e / (C / 8), pc = e % (C / 8);
        *(u32x4*)(w1_lds + r * W1S + pc * 8) = *(const u32x4*)(w1 + (int64_t)r * C + pc * 8);
    }
    for (int e = tid; e < C * H; e += MLP_THREADS) {
        const int c = e / H, hdn = e % H;
        w2_lds[c * W2S + (hdn & ~31) + perm32(hdn & 31)] = w2[(int64_t)c * H + hdn];
    }
    for (int e = tid; e < H; e += MLP_THREADS) b1_lds[e] = (float)b1[e];
    for (int e = tid; e < C; e += MLP_THREADS) b2_lds[e] = (float)b2[e];
    __syncthreads();

    constexpr int PIECES = 32 * C / 8;          // 16-byte pieces of a 32-row tile
    constexpr int IT = PIECES / PTV3_WAVE;      // per lane: 2 (C=32) or 4 (C=64)
    constexpr int PPR = C / 8;                  // pieces per row
    const int64_t n_tiles = (n + 31) / 32;
    for (int64_t tile = (int64_t)blockIdx.x * MLP_WAVES + wave; tile < n_tiles; tile += (int64_t)gridDim.x * MLP_WAVES) {
        const int64_t row0 = tile * 32;
        // ---- X tile: contiguous 16-byte pieces -> LDS -> operand registers (one row per lane)
        u32x4 xr[IT], rr[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            xr[it] = (u32x4){0, 0, 0, 0};
            rr[it] = (u32x4){0, 0, 0, 0};
            if (r < n) {
                xr[it] = *(const u32x4*)(x + r * C + (pidx % PPR) * 8);
                rr[it] = *(const u32x4*)(resid + r * C + (pidx % PPR) * 8);
            }
        }
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            *(u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8) = xr[it];
        }
        asm volatile("" ::: "memory");
        v8 xf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xf[ks] = __builtin_bit_cast(v8, *(const u32x4*)(xs + col * XSS + ks * 16 + hf * 8));
        asm volatile("" ::: "memory");

        f32x16 acc[OT];
#pragma unroll
        for (int o = 0; o < OT; ++o)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[o][v] = 0.f;

        for (int ht = 0; ht < H / 32; ++ht) {
            // hidden tile: 32 units x 32 rows
            f32x16 d;   // starts from the bias: the MFMAs' C operand
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(b1_lds + ht * 32 + 8 * g + 4 * hf);
#pragma unroll
                for (int q = 0; q < 4; ++q) d[4 * g + q] = bb[q];
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v8 wf = __builtin_bit_cast(v8, *(const u32x4*)(w1_lds + (ht * 32 + col) * W1S + ks * 16 + hf * 8));
                d = H16<T>::mfma(wf, xf[ks], d);
            }
            // round to storage precision as a separate fc1 would, GELU, round again
            uint32_t p[8];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                p[2 * g] = gelu_round_pack2<T>(d[4 * g], d[4 * g + 1]);
                p[2 * g + 1] = gelu_round_pack2<T>(d[4 * g + 2], d[4 * g + 3]);
            }
            const v8 pa = __builtin_bit_cast(v8, (u32x4){p[0], p[1], p[2], p[3]});
            const v8 pb = __builtin_bit_cast(v8, (u32x4){p[4], p[5], p[6], p[7]});
#pragma unroll
            for (int o = 0; o < OT; ++o) {
                const T* wrow = w2_lds + (o * 32 + col) * W2S + ht * 32 + hf * 16;
                acc[o] = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)wrow), pa, acc[o]);
                acc[o] = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(wrow + 8)), pb, acc[o]);
            }
        }
        // ---- epilogue: acc[o][v] is channel o*32 + 8*(v/4) + 4*hf + v%4 of row col. Add fc2's bias,
        // round as a separate fc2 would, back to contiguous pieces, add the residual, store.
#pragma unroll
        for (int o = 0; o < OT; ++o)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(b2_lds + o * 32 + 8 * g + 4 * hf);
                u32x2 pk = {H16<T>::pack2(acc[o][4 * g] + bb[0], acc[o][4 * g + 1] + bb[1]),
                            H16<T>::pack2(acc[o][4 * g + 2] + bb[2], acc[o][4 * g + 3] + bb[3])};
                *(u32x2*)(xs + col * XSS + o * 32 + 8 * g + 4 * hf) = pk;
            }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            const u32x4 y = *(const u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8);
            u32x4 o4;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                o4[k] = H16<T>::pack2(H16<T>::lo(y[k]) + H16<T>::lo(rr[it][k]), H16<T>::hi(y[k]) + H16<T>::hi(rr[it][k]));
            if (r < n) *(u32x4*)(out + r * C + (pidx % PPR) * 8) = o4;
        }
        asm volatile("" ::: "memory");
    }
}

template <typename T, int C>
int launch_mlp(const void* x, const void* resid, const void* w1, const void* b1, const void* w2, const void* b2,
               int64_t n, void* out, hipStream_t stream) {
    constexpr int H = 4 * C;
    const size_t lds = ((size_t)H * (C + PADH) + (size_t)C * (H + PADH)) * sizeof(T) + (size_t)(H + C) * sizeof(float) +
                       (size_t)MLP_WAVES * 32 * (C + PADH) * sizeof(T);
    auto kern = mlp_fused_kernel<T, C>;
    static LdsGrant grant_configured;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_configured)) return rc_;
    // persistent work-groups: weights are staged once per work-group, so no more of them than the
    // machine holds at a time (or than there are row tiles)
    const int64_t tiles = (n + 31) / 32;
    int64_t blocks = (tiles + MLP_WAVES - 1) / MLP_WAVES;
    const int64_t resident = lds > 80 * 1024 ? 256 : 512;
    if (blocks > resident) blocks = resident;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(MLP_THREADS), lds, stream, (const T*)x, (const T*)resid,
                       (const T*)w1, (const T*)b1, (const T*)w2, (const T*)b2, n, (T*)out);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

}  // namespace

// wide channels (128, 256, 512): mlpwide.hip
int mlp_wide_dispatch(const void* x, const void* resid, const void* w1, const void* b1, const void* w2, const void* b2,
                      int dtype, int64_t n, int channels, void* out, hipStream_t stream);

extern "C" int ptv3_mlp_fused(const void* x, const void* resid, const void* w1, const void* b1, const void* w2,
                              const void* b2, int dtype, int64_t n, int channels, int hidden, void* out,
                              void* stream_) {
    if (n < 0 || channels < 1 || hidden < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    const bool thin = channels == 32 || channels == 64, wide = channels == 128 || channels == 256 || channels == 512;
    if ((!thin && !wide) || hidden != 4 * channels) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !resid || !w1 || !b1 || !w2 || !b2 || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (wide) return mlp_wide_dispatch(x, resid, w1, b1, w2, b2, dtype, n, channels, out, stream);
    if (dtype == PTV3_F16) {
        if (channels == 32) return launch_mlp<_Float16, 32>(x, resid, w1, b1, w2, b2, n, out, stream);
        return launch_mlp<_Float16, 64>(x, resid, w1, b1, w2, b2, n, out, stream);
    }
    if (channels == 32) return launch_mlp<__bf16, 32>(x, resid, w1, b1, w2, b2, n, out, stream);
    return launch_mlp<__bf16, 64>(x, resid, w1, b1, w2, b2, n, out, stream);
}
