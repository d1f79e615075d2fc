// Fused head and tail of a transformer block for thin channels (C = 32 or 64, half precision).
//
// At these widths every dense layer of model.py:586-606 is bound by its N x C tensors going to HBM
// and back; the two kernels here keep a 32-row tile in registers across the whole chain.
//
//   head:  branch = cpe.1(conv)                       Linear C->C        (model.py:541-545)
//          feat   = shortcut + cpe.2(branch)          LayerNorm + residual (model.py:587-589)
//          qkv    = attn.qkv(norm1(feat))             LayerNorm + Linear C->3C (model.py:592-593, :450)
//          writes feat (N,C) and qkv (N,3C)
//   tail:  feat   = shortcut + attn.proj(attn_out)    Linear C->C + residual (model.py:485-487, :594-595)
//          out    = feat + mlp(norm2(feat))           LayerNorm, fc1, GELU, fc2, residual (model.py:599-602)
//          writes out (N,C)
//
// A wave owns 32 rows; all weights stay in LDS for the life of a persistent work-group. Products
// are taken transposed with v_mfma_f32_32x32x16 (rows = output channels, columns = points), so a
// lane holds, for ONE point, channels 8*(v/4) + 4*(lane/32) + v%4 of every 32-channel block: row
// statistics of a LayerNorm are a lane-local sum plus one exchange with lane^32, and the normalised
// values, converted to 16 bit, are directly the B operand of the next product, whose weight matrix
// is stored with its input axis in that register order. Intermediates are rounded to the storage
// type wherever the separate layers would have stored them. Row tiles move between global memory
// and registers as contiguous 16-byte pieces through a wave-private LDS buffer.
#include "rowtile.h"

namespace {

constexpr int BLK_THREADS = 512;
constexpr int BLK_WAVES = BLK_THREADS / PTV3_WAVE;
constexpr int BPAD = 8;   // halfs of padding per LDS row

// LayerNorm over the C = 32*OT channels of the row a lane pair holds; values come back rounded.
template <typename T, int OT>
__device__ __forceinline__ void ln_lane_pair(float (&val)[OT][16], float eps, const float* __restrict__ gamma,
                                             const float* __restrict__ beta, int hf) {
    constexpr float INV_C = 1.f / (32 * OT);
    float s = 0.f;
#pragma unroll
    for (int o = 0; o < OT; ++o)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += val[o][v];
    s += __shfl_xor(s, 32, PTV3_WAVE);
    const float mean = s * INV_C;
    float q = 0.f;
#pragma unroll
    for (int o = 0; o < OT; ++o)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float d = val[o][v] - mean;
            q = fmaf(d, d, q);
        }
    q += __shfl_xor(q, 32, PTV3_WAVE);
    const float rstd = rsqrtf(q * INV_C + eps);
#pragma unroll
    for (int o = 0; o < OT; ++o)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 gg = *(const f32x4*)(gamma + o * 32 + 8 * g + 4 * hf);
            const f32x4 bb = *(const f32x4*)(beta + o * 32 + 8 * g + 4 * hf);
#pragma unroll
            for (int k = 0; k < 4; ++k)
                val[o][4 * g + k] = H16<T>::round((val[o][4 * g + k] - mean) * rstd * gg[k] + bb[k]);
        }
}

// copy an (rows x C) weight matrix into LDS rows of stride `stride`; PERM stores the input axis of
// every 32-block in MFMA result-register order
template <typename T, bool PERM>
__device__ __forceinline__ void stage_weight(T* __restrict__ dst, const T* __restrict__ src, int rows, int c,
                                             int stride, int tid) {
    if (PERM) {
        for (int e = tid; e < rows * c; e += BLK_THREADS) {
            const int r = e / c, k = e % c;
            dst[r * stride + (k & ~31) + perm32(k & 31)] = src[(int64_t)r * c + k];
        }
    } else {
        const int ppr = c / 8;
        for (int e = tid; e < rows * ppr; e += BLK_THREADS) {
            const int r = e / ppr, pc = e % ppr;
            *(u32x4*)(dst + r * stride + pc * 8) = *(const u32x4*)(src + (int64_t)r * c + pc * 8);
        }
    }
}

template <typename T>
__device__ __forceinline__ void stage_vec(float* __restrict__ dst, const T* __restrict__ src, int len, int tid,
                                          float fill) {
    for (int e = tid; e < len; e += BLK_THREADS) dst[e] = src ? (float)src[e] : fill;
}

template <typename T, int C>
__global__ __launch_bounds__(BLK_THREADS, 2) void block_head_kernel(
    const T* __restrict__ conv, const T* __restrict__ shortcut, const T* __restrict__ wc,
    const T* __restrict__ bc, const T* __restrict__ gc, const T* __restrict__ bec, float eps_c,
    const T* __restrict__ g1, const T* __restrict__ be1, float eps_1, const T* __restrict__ wq,
    const T* __restrict__ bq, int64_t n, T* __restrict__ feat, T* __restrict__ qkv) {
    typedef typename H16<T>::v8 v8;
    constexpr int KS = C / 16, OT = C / 32, QT = 3 * C / 32;
    constexpr int WS = C + BPAD;      // weight row stride (halfs)
    constexpr int XSS = 64 + BPAD;    // tile buffer row stride: wide enough for 64 output channels
    extern __shared__ __align__(16) unsigned char blk_smem[];
    T* wc_lds = (T*)blk_smem;                    // [C][WS]
    T* wq_lds = wc_lds + C * WS;                 // [3C][WS], input axis in register order
    float* bc_lds = (float*)(wq_lds + 3 * C * WS);
    float* gc_lds = bc_lds + C;
    float* bec_lds = gc_lds + C;
    float* g1_lds = bec_lds + C;
    float* be1_lds = g1_lds + C;
    float* bq_lds = be1_lds + C;                 // [3C]
    T* xs_all = (T*)(bq_lds + 3 * C);            // [waves][32][XSS]

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    T* xs = xs_all + wave * (32 * XSS);

    stage_weight<T, false>(wc_lds, wc, C, C, WS, tid);
    stage_weight<T, true>(wq_lds, wq, 3 * C, C, WS, tid);
    stage_vec<T>(bc_lds, bc, C, tid, 0.f);
    stage_vec<T>(gc_lds, gc, C, tid, 1.f);
    stage_vec<T>(bec_lds, bec, C, tid, 0.f);
    stage_vec<T>(g1_lds, g1, C, tid, 1.f);
    stage_vec<T>(be1_lds, be1, C, tid, 0.f);
    stage_vec<T>(bq_lds, bq, 3 * C, tid, 0.f);
    __syncthreads();

    constexpr int PPR = C / 8;                       // 16-byte pieces per row
    constexpr int IT = 32 * PPR / PTV3_WAVE;         // pieces per lane: 2 (C=32) or 4 (C=64)
    const int64_t n_tiles = (n + 31) / 32;
    for (int64_t tile = (int64_t)blockIdx.x * BLK_WAVES + wave; tile < n_tiles; tile += (int64_t)gridDim.x * BLK_WAVES) {
        const int64_t row0 = tile * 32;
        u32x4 xr[IT], rr[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            xr[it] = (u32x4){0, 0, 0, 0};
            rr[it] = (u32x4){0, 0, 0, 0};
            if (r < n) {
                xr[it] = *(const u32x4*)(conv + r * C + (pidx % PPR) * 8);
                rr[it] = *(const u32x4*)(shortcut + r * C + (pidx % PPR) * 8);
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
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            *(u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8) = rr[it];
        }
        asm volatile("" ::: "memory");

        // ---- branch = cpe.1(conv), rounded; then cpe.2
        float y[OT][16];
#pragma unroll
        for (int o = 0; o < OT; ++o) {
            f32x16 d;
#pragma unroll
            for (int v = 0; v < 16; ++v) d[v] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v8 wf = __builtin_bit_cast(v8, *(const u32x4*)(wc_lds + (o * 32 + col) * WS + ks * 16 + hf * 8));
                d = H16<T>::mfma(wf, xf[ks], d);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(bc_lds + o * 32 + 8 * g + 4 * hf);
#pragma unroll
                for (int k = 0; k < 4; ++k) y[o][4 * g + k] = H16<T>::round(d[4 * g + k] + bb[k]);
            }
        }
        ln_lane_pair<T, OT>(y, eps_c, gc_lds, bec_lds, hf);
        // ---- feat = shortcut + that, rounded; parked in the tile buffer for the piece-wise store
#pragma unroll
        for (int o = 0; o < OT; ++o)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                T* cell = xs + col * XSS + o * 32 + 8 * g + 4 * hf;
                const u32x2 sc = *(const u32x2*)cell;
                y[o][4 * g + 0] = H16<T>::round(y[o][4 * g + 0] + H16<T>::lo(sc[0]));
                y[o][4 * g + 1] = H16<T>::round(y[o][4 * g + 1] + H16<T>::hi(sc[0]));
                y[o][4 * g + 2] = H16<T>::round(y[o][4 * g + 2] + H16<T>::lo(sc[1]));
                y[o][4 * g + 3] = H16<T>::round(y[o][4 * g + 3] + H16<T>::hi(sc[1]));
                *(u32x2*)cell = (u32x2){H16<T>::pack2(y[o][4 * g], y[o][4 * g + 1]),
                                        H16<T>::pack2(y[o][4 * g + 2], y[o][4 * g + 3])};
            }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            const u32x4 f4 = *(const u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8);
            if (r < n) *(u32x4*)(feat + r * C + (pidx % PPR) * 8) = f4;
        }
        asm volatile("" ::: "memory");

        // ---- norm1, then qkv two 32-channel tiles (64 output channels) at a time
        ln_lane_pair<T, OT>(y, eps_1, g1_lds, be1_lds, hf);
        v8 xn[2 * OT];
#pragma unroll
        for (int o = 0; o < OT; ++o) {
            uint32_t p[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) p[k] = H16<T>::pack2(y[o][2 * k], y[o][2 * k + 1]);
            xn[2 * o] = __builtin_bit_cast(v8, (u32x4){p[0], p[1], p[2], p[3]});
            xn[2 * o + 1] = __builtin_bit_cast(v8, (u32x4){p[4], p[5], p[6], p[7]});
        }
#pragma unroll
        for (int grp = 0; grp < QT; grp += 2) {
            const int nt = (QT - grp) < 2 ? (QT - grp) : 2;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (t >= nt) break;
                f32x16 d;
#pragma unroll
                for (int v = 0; v < 16; ++v) d[v] = 0.f;
                const T* wrow = wq_lds + ((grp + t) * 32 + col) * WS + hf * 16;
#pragma unroll
                for (int o = 0; o < OT; ++o) {
                    d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(wrow + o * 32)), xn[2 * o], d);
                    d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(wrow + o * 32 + 8)), xn[2 * o + 1], d);
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 bb = *(const f32x4*)(bq_lds + (grp + t) * 32 + 8 * g + 4 * hf);
                    *(u32x2*)(xs + col * XSS + t * 32 + 8 * g + 4 * hf) =
                        (u32x2){H16<T>::pack2(d[4 * g] + bb[0], d[4 * g + 1] + bb[1]),
                                H16<T>::pack2(d[4 * g + 2] + bb[2], d[4 * g + 3] + bb[3])};
                }
            }
            asm volatile("" ::: "memory");
            const int ppr_g = nt * 4;                        // pieces per row of this group
            const int its = 32 * ppr_g / PTV3_WAVE;          // 4 or 2
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                if (it >= its) break;
                const int pidx = it * PTV3_WAVE + lane;
                const int rr_ = pidx / ppr_g, pc = pidx % ppr_g;
                const int64_t r = row0 + rr_;
                const u32x4 q4 = *(const u32x4*)(xs + rr_ * XSS + pc * 8);
                if (r < n) *(u32x4*)(qkv + r * (3 * C) + grp * 32 + pc * 8) = q4;
            }
            asm volatile("" ::: "memory");
        }
    }
}

template <typename T, int C>
__global__ __launch_bounds__(BLK_THREADS, 2) void block_tail_kernel(
    const T* __restrict__ attn, const T* __restrict__ shortcut, const T* __restrict__ wp,
    const T* __restrict__ bp, const T* __restrict__ g2, const T* __restrict__ be2, float eps_2,
    const T* __restrict__ w1, const T* __restrict__ b1, const T* __restrict__ w2, const T* __restrict__ b2,
    int64_t n, T* __restrict__ out) {
    typedef typename H16<T>::v8 v8;
    constexpr int H = 4 * C;
    constexpr int KS = C / 16, OT = C / 32;
    constexpr int WS = C + BPAD;
    constexpr int W2S = H + BPAD;
    constexpr int XSS = C + BPAD;
    extern __shared__ __align__(16) unsigned char blk_smem[];
    T* wp_lds = (T*)blk_smem;                    // [C][WS]
    T* w1_lds = wp_lds + C * WS;                 // [H][WS], input axis in register order
    T* w2_lds = w1_lds + H * WS;                 // [C][W2S], hidden axis in register order
    float* bp_lds = (float*)(w2_lds + C * W2S);
    float* g2_lds = bp_lds + C;
    float* be2_lds = g2_lds + C;
    float* b2_lds = be2_lds + C;
    float* b1_lds = b2_lds + C;                  // [H]
    T* xs_all = (T*)(b1_lds + H);                // [waves][32][XSS]

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    T* xs = xs_all + wave * (32 * XSS);

    stage_weight<T, false>(wp_lds, wp, C, C, WS, tid);
    stage_weight<T, true>(w1_lds, w1, H, C, WS, tid);
    stage_weight<T, true>(w2_lds, w2, C, H, W2S, tid);
    stage_vec<T>(bp_lds, bp, C, tid, 0.f);
    stage_vec<T>(g2_lds, g2, C, tid, 1.f);
    stage_vec<T>(be2_lds, be2, C, tid, 0.f);
    stage_vec<T>(b2_lds, b2, C, tid, 0.f);
    stage_vec<T>(b1_lds, b1, H, tid, 0.f);
    __syncthreads();

    constexpr int PPR = C / 8;
    constexpr int IT = 32 * PPR / PTV3_WAVE;
    const int64_t n_tiles = (n + 31) / 32;
    for (int64_t tile = (int64_t)blockIdx.x * BLK_WAVES + wave; tile < n_tiles; tile += (int64_t)gridDim.x * BLK_WAVES) {
        const int64_t row0 = tile * 32;
        u32x4 xr[IT], rr[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            xr[it] = (u32x4){0, 0, 0, 0};
            rr[it] = (u32x4){0, 0, 0, 0};
            if (r < n) {
                xr[it] = *(const u32x4*)(attn + r * C + (pidx % PPR) * 8);
                rr[it] = *(const u32x4*)(shortcut + r * C + (pidx % PPR) * 8);
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
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            *(u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8) = rr[it];
        }
        asm volatile("" ::: "memory");

        // ---- feat = shortcut + proj(attn), both rounded as the separate layers round them
        float y[OT][16];
        uint32_t fp[OT][8];   // feat, kept packed for the last residual add
#pragma unroll
        for (int o = 0; o < OT; ++o) {
            f32x16 d;
#pragma unroll
            for (int v = 0; v < 16; ++v) d[v] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const v8 wf = __builtin_bit_cast(v8, *(const u32x4*)(wp_lds + (o * 32 + col) * WS + ks * 16 + hf * 8));
                d = H16<T>::mfma(wf, xf[ks], d);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(bp_lds + o * 32 + 8 * g + 4 * hf);
                const u32x2 sc = *(const u32x2*)(xs + col * XSS + o * 32 + 8 * g + 4 * hf);
                y[o][4 * g + 0] = H16<T>::round(H16<T>::round(d[4 * g + 0] + bb[0]) + H16<T>::lo(sc[0]));
                y[o][4 * g + 1] = H16<T>::round(H16<T>::round(d[4 * g + 1] + bb[1]) + H16<T>::hi(sc[0]));
                y[o][4 * g + 2] = H16<T>::round(H16<T>::round(d[4 * g + 2] + bb[2]) + H16<T>::lo(sc[1]));
                y[o][4 * g + 3] = H16<T>::round(H16<T>::round(d[4 * g + 3] + bb[3]) + H16<T>::hi(sc[1]));
                fp[o][2 * g] = H16<T>::pack2(y[o][4 * g], y[o][4 * g + 1]);
                fp[o][2 * g + 1] = H16<T>::pack2(y[o][4 * g + 2], y[o][4 * g + 3]);
            }
        }
        asm volatile("" ::: "memory");
        // ---- norm2 -> operand of fc1
        ln_lane_pair<T, OT>(y, eps_2, g2_lds, be2_lds, hf);
        v8 xn[2 * OT];
#pragma unroll
        for (int o = 0; o < OT; ++o) {
            uint32_t p[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) p[k] = H16<T>::pack2(y[o][2 * k], y[o][2 * k + 1]);
            xn[2 * o] = __builtin_bit_cast(v8, (u32x4){p[0], p[1], p[2], p[3]});
            xn[2 * o + 1] = __builtin_bit_cast(v8, (u32x4){p[4], p[5], p[6], p[7]});
        }

        f32x16 acc[OT];
#pragma unroll
        for (int o = 0; o < OT; ++o)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[o][v] = 0.f;

        for (int ht = 0; ht < H / 32; ++ht) {
            // the accumulator starts from fc1's bias (the MFMA's C operand) instead of adding it afterwards
            f32x16 d;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(b1_lds + ht * 32 + 8 * g + 4 * hf);
#pragma unroll
                for (int q = 0; q < 4; ++q) d[4 * g + q] = bb[q];
            }
            const T* w1row = w1_lds + (ht * 32 + col) * WS + hf * 16;
#pragma unroll
            for (int o = 0; o < OT; ++o) {
                d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(w1row + o * 32)), xn[2 * o], d);
                d = H16<T>::mfma(__builtin_bit_cast(v8, *(const u32x4*)(w1row + o * 32 + 8)), xn[2 * o + 1], d);
            }
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
        // ---- out = feat + (fc2 + bias, rounded), back to contiguous pieces
#pragma unroll
        for (int o = 0; o < OT; ++o)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 bb = *(const f32x4*)(b2_lds + o * 32 + 8 * g + 4 * hf);
                const uint32_t f0 = fp[o][2 * g], f1 = fp[o][2 * g + 1];
                const float o0 = H16<T>::round(acc[o][4 * g + 0] + bb[0]) + H16<T>::lo(f0);
                const float o1 = H16<T>::round(acc[o][4 * g + 1] + bb[1]) + H16<T>::hi(f0);
                const float o2 = H16<T>::round(acc[o][4 * g + 2] + bb[2]) + H16<T>::lo(f1);
                const float o3 = H16<T>::round(acc[o][4 * g + 3] + bb[3]) + H16<T>::hi(f1);
                *(u32x2*)(xs + col * XSS + o * 32 + 8 * g + 4 * hf) =
                    (u32x2){H16<T>::pack2(o0, o1), H16<T>::pack2(o2, o3)};
            }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int pidx = it * PTV3_WAVE + lane;
            const int64_t r = row0 + pidx / PPR;
            const u32x4 o4 = *(const u32x4*)(xs + (pidx / PPR) * XSS + (pidx % PPR) * 8);
            if (r < n) *(u32x4*)(out + r * C + (pidx % PPR) * 8) = o4;
        }
        asm volatile("" ::: "memory");
    }
}

int64_t persistent_blocks(int64_t n, size_t lds) {
    const int64_t tiles = (n + 31) / 32;
    int64_t blocks = (tiles + BLK_WAVES - 1) / BLK_WAVES;
    const int64_t resident = lds > 80 * 1024 ? 256 : 512;
    return blocks > resident ? resident : blocks;
}

template <typename T, int C>
int launch_head(const void* conv, const void* shortcut, const void* wc, const void* bc, const void* gc,
                const void* bec, float eps_c, const void* g1, const void* be1, float eps_1, const void* wq,
                const void* bq, int64_t n, void* feat, void* qkv, hipStream_t stream) {
    const size_t lds = ((size_t)4 * C * (C + BPAD)) * sizeof(T) + (size_t)(8 * C) * sizeof(float) +
                       (size_t)BLK_WAVES * 32 * (64 + BPAD) * sizeof(T);
    auto kern = block_head_kernel<T, C>;
    static LdsGrant grant_configured;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_configured)) return rc_;
    hipLaunchKernelGGL(kern, dim3((unsigned)persistent_blocks(n, lds)), dim3(BLK_THREADS), lds, stream,
                       (const T*)conv, (const T*)shortcut, (const T*)wc, (const T*)bc, (const T*)gc, (const T*)bec,
                       eps_c, (const T*)g1, (const T*)be1, eps_1, (const T*)wq, (const T*)bq, n, (T*)feat, (T*)qkv);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

template <typename T, int C>
int launch_tail(const void* attn, const void* shortcut, const void* wp, const void* bp, const void* g2,
                const void* be2, float eps_2, const void* w1, const void* b1, const void* w2, const void* b2,
                int64_t n, void* out, hipStream_t stream) {
    constexpr int H = 4 * C;
    const size_t lds = ((size_t)C * (C + BPAD) + (size_t)H * (C + BPAD) + (size_t)C * (H + BPAD)) * sizeof(T) +
                       (size_t)(4 * C + H) * sizeof(float) + (size_t)BLK_WAVES * 32 * (C + BPAD) * sizeof(T);
    auto kern = block_tail_kernel<T, C>;
    static LdsGrant grant_configured;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_configured)) return rc_;
    hipLaunchKernelGGL(kern, dim3((unsigned)persistent_blocks(n, lds)), dim3(BLK_THREADS), lds, stream,
                       (const T*)attn, (const T*)shortcut, (const T*)wp, (const T*)bp, (const T*)g2, (const T*)be2,
                       eps_2, (const T*)w1, (const T*)b1, (const T*)w2, (const T*)b2, n, (T*)out);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

}  // namespace

extern "C" int ptv3_block_head_fused(const void* conv, const void* shortcut, const void* w_cpe, const void* b_cpe,
                                     const void* ln_cpe_gamma, const void* ln_cpe_beta, float ln_cpe_eps,
                                     const void* ln1_gamma, const void* ln1_beta, float ln1_eps, const void* w_qkv,
                                     const void* b_qkv, int dtype, int64_t n, int channels, void* feat, void* qkv,
                                     void* stream_) {
    if (n < 0 || channels < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (channels != 32 && channels != 64) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!conv || !shortcut || !w_cpe || !w_qkv || !feat || !qkv) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
#define PTV3_HEAD(T, C)                                                                                      \
    return launch_head<T, C>(conv, shortcut, w_cpe, b_cpe, ln_cpe_gamma, ln_cpe_beta, ln_cpe_eps, ln1_gamma, \
                             ln1_beta, ln1_eps, w_qkv, b_qkv, n, feat, qkv, stream)
    if (dtype == PTV3_F16) {
        if (channels == 32) PTV3_HEAD(_Float16, 32);
        PTV3_HEAD(_Float16, 64);
    }
    if (channels == 32) PTV3_HEAD(__bf16, 32);
    PTV3_HEAD(__bf16, 64);
#undef PTV3_HEAD
}

extern "C" int ptv3_block_tail_fused(const void* attn, const void* shortcut, const void* w_proj, const void* b_proj,
                                     const void* ln2_gamma, const void* ln2_beta, float ln2_eps, const void* w1,
                                     const void* b1, const void* w2, const void* b2, int dtype, int64_t n,
                                     int channels, int hidden, void* out, void* stream_) {
    if (n < 0 || channels < 1 || hidden < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if ((channels != 32 && channels != 64) || hidden != 4 * channels) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!attn || !shortcut || !w_proj || !w1 || !w2 || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
#define PTV3_TAIL(T, C)                                                                                     \
    return launch_tail<T, C>(attn, shortcut, w_proj, b_proj, ln2_gamma, ln2_beta, ln2_eps, w1, b1, w2, b2, n, out, \
                             stream)
    if (dtype == PTV3_F16) {
        if (channels == 32) PTV3_TAIL(_Float16, 32);
        PTV3_TAIL(_Float16, 64);
    }
    if (channels == 32) PTV3_TAIL(__bf16, 32);
    PTV3_TAIL(__bf16, 64);
#undef PTV3_TAIL
}
