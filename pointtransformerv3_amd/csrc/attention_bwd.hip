// Backward of the serialized patch attention (head_dim 16), with the gathers either side of it.
//
// What autograd derives for model.py:456-484 of the reference (the backward of
// flash_attn_varlen_qkvpacked_func at :476-482, and of the row gathers qkv[order] and feat[inverse]
// around it): given dO, per sequence and head, with P = softmax(scale * Q K^T) and D_i = <dO_i, O_i>,
//     dV = P^T dO,   dS = P o (dO V^T - D),   dQ = scale * dS K,   dK = scale * dS^T Q.
// Filler slots of a padded sequence repeat rows of the patch before; as queries they receive no
// gradient, as keys they do, and it is added to the row they repeat.
//
// Half precision, two kernels per (sequence, head), both on v_mfma_f32_32x32x16 with the products
// transposed as in the forward kernel so that a lane owns one query (first kernel) or one key
// (second kernel) and row-wise quantities stay lane-local:
//   1. queries: K, V (rows) and K^T (transposed) in LDS. A first sweep over the keys gives the
//      log-sum-exp of every query row, a second one P = 2^(S - lse) directly (the -lse and -D
//      enter through the MFMAs' C operands), dS and dQ^T += K^T dS^T. lse and D go to a workspace.
//   2. keys: Q, dO (rows), Q^T, dO^T (transposed), -lse and -D in LDS; per 32-key tile
//      dV^T += dO^T P and dK^T += Q^T dS over all queries.
// fp32: one thread per query / per key, operands staged through LDS in chunks.
#include "attn_half.h"

namespace {

constexpr int BWD_THREADS = 512;    // keys kernel: 8 waves, two key tiles each per sweep
constexpr int BWD_WAVES = BWD_THREADS / PTV3_WAVE;
constexpr int BWQ_THREADS = 1024;   // queries kernel: 16 waves, four per SIMD
constexpr int BWQ_WAVES = BWQ_THREADS / PTV3_WAVE;
constexpr float LN2 = 0.6931471805599453f;
constexpr float LOG2E = 1.4426950408889634f;

// Stages `count` slots of 16 channels into LDS: as rows of 32 B (ROWS) and / or transposed, 16
// rows of t_stride bytes with the slot axis permuted inside 32-blocks to the order in which the
// MFMA result registers hold them (TRANS). fetch(slot, half) returns channels [8 half, 8 half + 8).
template <bool ROWS, bool TRANS, int THREADS, typename F>
__device__ __forceinline__ void stage16(int tid, int count, F fetch, unsigned char* rows_lds, unsigned char* t_lds,
                                        int t_stride) {
    for (int e0 = tid; e0 < count * 2; e0 += 4 * THREADS) {
        u32x4 w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = e0 + j * THREADS;
            w[j] = (u32x4){0, 0, 0, 0};
            if (e < count * 2) w[j] = fetch(e >> 1, e & 1);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = e0 + j * THREADS;
            if (e >= count * 2) break;
            const int key = e >> 1, half8 = e & 1;
            if (ROWS) *(u32x4*)(rows_lds + key * 32 + half8 * 16) = w[j];
            if (TRANS) {
                const int pos = (key & ~31) + vt_pos(key & 31);
                unsigned char* t = t_lds + (size_t)(half8 * 8) * t_stride + pos * 2;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    *(uint16_t*)(t + (size_t)(2 * c) * t_stride) = (uint16_t)(w[j][c] & 0xffffu);
                    *(uint16_t*)(t + (size_t)(2 * c + 1) * t_stride) = (uint16_t)(w[j][c] >> 16);
                }
            }
        }
    }
}

template <typename T>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b) {
    typedef typename Half<T>::v8 v8;
    const v8 x = __builtin_bit_cast(v8, a), y = __builtin_bit_cast(v8, b);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = fmaf((float)x[i], (float)y[i], s);
    return s;
}

template <typename T>
__device__ __forceinline__ typename Half<T>::v8 pack8(const float* f) {
    typedef typename Half<T>::v8 v8;
    return __builtin_bit_cast(v8, (u32x4){Half<T>::pack2(f[0], f[1]), Half<T>::pack2(f[2], f[3]),
                                          Half<T>::pack2(f[4], f[5]), Half<T>::pack2(f[6], f[7])});
}

__device__ __forceinline__ f32x16 splat16(float x) {
    f32x16 r;
#pragma unroll
    for (int v = 0; v < 16; ++v) r[v] = x;
    return r;
}

// Work-group id -> (item, part of parts): the first full_items work-groups take one (sequence, head) item each;
// the items of the last, partly filled round of resident work-groups are cut into `split` ranges of tiles, one
// work-group each, so that the round is short (every range stages the sequence again).
__device__ __forceinline__ void item_of_block(int full_items, int split, int* item, int* part, int* parts) {
    if ((int)blockIdx.x < full_items) {
        *item = xcd_chunked_id(blockIdx.x, full_items);   // heads that share cache lines meet in one L2
        *part = 0;
        *parts = 1;
    } else {
        const int r = blockIdx.x - full_items;
        *item = full_items + r / split;
        *part = r % split;
        *parts = split;
    }
}

// ---- kernel 1: one work-group per (sequence, head), a wave per 32-query tile
template <typename T, bool HAVE_LSE, bool DROP>
__global__ __launch_bounds__(BWQ_THREADS) void attn_bwd_q_kernel(
    const T* __restrict__ qkv, const T* __restrict__ out, const T* __restrict__ dout, int channels, int heads,
    const int32_t* __restrict__ slot_src, const int32_t* __restrict__ slot_dst,
    const int32_t* __restrict__ cu_seqlens, int lds_keys, float scale, int64_t n_pad, T* __restrict__ dqkv,
    float* lse_ws, float* __restrict__ d_ws, int full_items, int split, Dropout drop) {
    typedef typename Half<T>::v8 v8;
    extern __shared__ __align__(16) unsigned char smem[];
    // K rows, V rows, K^T, 96 B of zeros
    const int kt_stride = lds_keys * 2 + VT_PAD_BYTES;
    unsigned char* k_lds = smem;
    unsigned char* v_lds = k_lds + (size_t)lds_keys * 32;
    unsigned char* kt_lds = v_lds + (size_t)lds_keys * 32;
    unsigned char* zero_lds = kt_lds + (size_t)HD * kt_stride;

    int item, part, parts;
    item_of_block(full_items, split, &item, &part, &parts);
    const int seq = item / heads, head = item % heads;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (len <= 0) return;
    const int len64 = (len + 63) & ~63;
    const int n_pairs = len64 / 64;
    const int tid = threadIdx.x;
    const int64_t row_stride = 3 * (int64_t)channels;

    if (tid < 24) ((uint32_t*)zero_lds)[tid] = 0u;
    stage16<true, true, BWQ_THREADS>(tid, len64, [&](int key, int half8) {
        u32x4 w = {0, 0, 0, 0};
        if (key < len) w = *(const u32x4*)(qkv + (int64_t)slot_src[s0 + key] * row_stride + channels + head * HD + half8 * 8);
        return w;
    }, k_lds, kt_lds, kt_stride);
    stage16<true, false, BWQ_THREADS>(tid, len64, [&](int key, int half8) {
        u32x4 w = {0, 0, 0, 0};
        if (key < len) w = *(const u32x4*)(qkv + (int64_t)slot_src[s0 + key] * row_stride + 2 * channels + head * HD + half8 * 8);
        return w;
    }, v_lds, nullptr, 0);
    __syncthreads();

    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int n_qtiles = (len + 31) / 32;
    const bool ragged = (len & 63) != 0;
    const float scale_log2e = scale * LOG2E;
    const unsigned char* k_base = k_lds + col * 32 + hf * 16;
    const unsigned char* v_base = v_lds + col * 32 + hf * 16;
    // A operand rows of dQ^T += K^T dS^T: rows d < 16 read K^T and advance 128 B per step, the others zeros
    const unsigned char* kt_base = col < HD ? kt_lds + (size_t)col * kt_stride + hf * 32 : zero_lds;
    const int kt_step = col < HD ? 128 : 0;

    const int qt_lo = (int)((int64_t)part * n_qtiles / parts), qt_hi = (int)((int64_t)(part + 1) * n_qtiles / parts);
    for (int qt = qt_lo + wave; qt < qt_hi; qt += BWQ_WAVES) {
        const int qi = qt * 32 + col;
        int dst = -1;
        u32x4 qreg = {0, 0, 0, 0}, doreg = {0, 0, 0, 0}, oreg = {0, 0, 0, 0};
        if (qi < len) {
            dst = slot_dst[s0 + qi];
            if (dst >= 0) {   // a real slot: the row it reads is the row it writes
                qreg = *(const u32x4*)(qkv + (int64_t)dst * row_stride + head * HD + hf * 8);
                doreg = *(const u32x4*)(dout + (int64_t)dst * channels + head * HD + hf * 8);
                oreg = *(const u32x4*)(out + (int64_t)dst * channels + head * HD + hf * 8);
            }
        }
        if (__ballot(dst >= 0) == 0) continue;   // filler slots only: no gradient arrives here
        float dsum = dot8<T>(doreg, oreg);
        dsum += __shfl_xor(dsum, 32, PTV3_WAVE);
        const v8 qfrag = __builtin_bit_cast(v8, scale8<T>(qreg, scale_log2e));   // scores in log2 units
        const v8 dofrag = __builtin_bit_cast(v8, doreg);
        const uint32_t hq = DROP ? drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + qi)) : 0u;

        // log-sum-exp of the query's score row: kept by the forward pass, or a first sweep over the keys
        // (this lane sees half of them)
        const f32x16 zero = splat16(0.f);
        float lse = 0.f;
        if (HAVE_LSE) {
            if (dst >= 0) lse = lse_ws[(int64_t)head * n_pad + s0 + qi];
        } else {
            float m = -INFINITY, l = 0.f;
            for (int kp = 0; kp < n_pairs; ++kp) {
                const v8 k0 = __builtin_bit_cast(v8, *(const u32x4*)(k_base + (size_t)kp * 64 * 32));
                const v8 k1 = __builtin_bit_cast(v8, *(const u32x4*)(k_base + (size_t)kp * 64 * 32 + 32 * 32));
                f32x16 sa = Half<T>::mfma(k0, qfrag, zero);
                f32x16 sb = Half<T>::mfma(k1, qfrag, zero);
                if (ragged && kp == n_pairs - 1) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = kp * 64 + 8 * (v >> 2) + 4 * hf + (v & 3);
                        if (key >= len) sa[v] = -INFINITY;
                        if (key + 32 >= len) sb[v] = -INFINITY;
                    }
                }
                float mx = fmaxf(sa[0], sb[0]);
#pragma unroll
                for (int v = 1; v < 16; ++v) mx = fmaxf(mx, fmaxf(sa[v], sb[v]));
                const float m_new = fmaxf(m, mx);
                const float ms = m_new == -INFINITY ? 0.f : m_new;
                float add = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) add += __builtin_amdgcn_exp2f(sa[v] - ms) + __builtin_amdgcn_exp2f(sb[v] - ms);
                l = l * __builtin_amdgcn_exp2f(m - ms) + add;
                m = m_new;
            }
            {
                const float mo = __shfl_xor(m, 32, PTV3_WAVE), lo = __shfl_xor(l, 32, PTV3_WAVE);
                const float mm = fmaxf(m, mo);
                const float ms = mm == -INFINITY ? 0.f : mm;
                l = l * __builtin_amdgcn_exp2f(m - ms) + lo * __builtin_amdgcn_exp2f(mo - ms);
                m = ms;
            }
            lse = dst >= 0 ? m + __builtin_amdgcn_logf(l) : 0.f;   // log2 units
        }

        // second sweep: P, dS and dQ^T
        const f32x16 c_lse = splat16(-lse), c_d = splat16(-dsum);
        f32x16 acc = zero;
        const unsigned char* kt_ptr = kt_base;
        for (int kp = 0; kp < n_pairs; ++kp) {
            // the two 32-key halves of the step one after the other: fewer values alive at a time
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const v8 kf = __builtin_bit_cast(v8, *(const u32x4*)(k_base + (size_t)kp * 64 * 32 + h * 32 * 32));
                const v8 vf = __builtin_bit_cast(v8, *(const u32x4*)(v_base + (size_t)kp * 64 * 32 + h * 32 * 32));
                f32x16 sc = Half<T>::mfma(kf, qfrag, c_lse);        // S - lse
                const f32x16 dp = Half<T>::mfma(vf, dofrag, DROP ? zero : c_d);   // dP - D (dP alone with dropout)
                const u32x4 kt0 = *(const u32x4*)(kt_ptr + 64 * h);
                const u32x4 kt1 = *(const u32x4*)(kt_ptr + 64 * h + 16);
                if (ragged && kp == n_pairs - 1) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        if (kp * 64 + 32 * h + 8 * (v >> 2) + 4 * hf + (v & 3) >= len) sc[v] = -INFINITY;
                }
                float ds[16];
                if (DROP) {
                    // the dropped probabilities pass no gradient on: dS = P o (mask o dP / (1 - p) - D)
                    const uint32_t k0s = (uint32_t)s0 + (uint32_t)kp * 64u + 32u * (uint32_t)h + 4u * (uint32_t)hf;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const bool keep = drop_keep(hq, k0s + 8u * (uint32_t)(v >> 2) + (uint32_t)(v & 3), drop.threshold);
                        ds[v] = __builtin_amdgcn_exp2f(sc[v]) * ((keep ? dp[v] * drop.inv_keep : 0.f) - dsum);
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) ds[v] = __builtin_amdgcn_exp2f(sc[v]) * dp[v];
                }
                acc = Half<T>::mfma(__builtin_bit_cast(v8, kt0), pack8<T>(ds), acc);
                acc = Half<T>::mfma(__builtin_bit_cast(v8, kt1), pack8<T>(ds + 8), acc);
            }
            kt_ptr += kt_step;
        }
        if (dst >= 0) {
            // acc[v], v < 8: channel d = 8 (v / 4) + 4 hf + v % 4 of this lane's query
            T* o = dqkv + (int64_t)dst * row_stride + head * HD + 4 * hf;
            u32x2 lo = {Half<T>::pack2(acc[0] * scale, acc[1] * scale), Half<T>::pack2(acc[2] * scale, acc[3] * scale)};
            u32x2 hi = {Half<T>::pack2(acc[4] * scale, acc[5] * scale), Half<T>::pack2(acc[6] * scale, acc[7] * scale)};
            *(u32x2*)o = lo;
            *(u32x2*)(o + 8) = hi;
            if (hf == 0) {
                if (!HAVE_LSE) lse_ws[(int64_t)head * n_pad + s0 + qi] = lse;
                d_ws[(int64_t)head * n_pad + s0 + qi] = dsum;
            }
        }
    }
}

// ---- kernel 2: one work-group per (sequence, head), a wave per 32-key tile
template <typename T, bool DROP>
__global__ __launch_bounds__(BWD_THREADS) void attn_bwd_kv_kernel(
    const T* __restrict__ qkv, const T* __restrict__ dout, int channels, int heads,
    const int32_t* __restrict__ slot_src, const int32_t* __restrict__ slot_dst,
    const int32_t* __restrict__ cu_seqlens, int lds_keys, float scale, int64_t n_pad,
    const float* __restrict__ lse_ws, const float* __restrict__ d_ws, T* __restrict__ dqkv, T* __restrict__ fill,
    int full_items, int split, Dropout drop) {
    typedef typename Half<T>::v8 v8;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char smem[];
    const int t_stride = lds_keys * 2 + VT_PAD_BYTES;
    unsigned char* q_lds = smem;                                      // Q * scale * log2(e), rows
    unsigned char* do_lds = q_lds + (size_t)lds_keys * 32;            // dO rows
    unsigned char* qt_lds = do_lds + (size_t)lds_keys * 32;           // the same two, transposed
    unsigned char* dot_lds = qt_lds + (size_t)HD * t_stride;
    float* nlse_lds = (float*)(dot_lds + (size_t)HD * t_stride);      // -lse (log2 units), -D per query slot
    float* nd_lds = nlse_lds + lds_keys;
    unsigned char* zero_lds = (unsigned char*)(nd_lds + lds_keys);

    int item, part, parts;
    item_of_block(full_items, split, &item, &part, &parts);
    const int seq = item / heads, head = item % heads;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (len <= 0) return;
    const int len64 = (len + 63) & ~63;
    const int n_pairs = len64 / 64;
    const int tid = threadIdx.x;
    const int64_t row_stride = 3 * (int64_t)channels;
    const float scale_log2e = scale * LOG2E;

    if (tid < 24) ((uint32_t*)zero_lds)[tid] = 0u;
    stage16<true, true, BWD_THREADS>(tid, len64, [&](int key, int half8) {
        u32x4 w = {0, 0, 0, 0};
        if (key < len)
            w = scale8<T>(*(const u32x4*)(qkv + (int64_t)slot_src[s0 + key] * row_stride + head * HD + half8 * 8), scale_log2e);
        return w;
    }, q_lds, qt_lds, t_stride);
    stage16<true, true, BWD_THREADS>(tid, len64, [&](int key, int half8) {
        u32x4 w = {0, 0, 0, 0};
        if (key < len) {
            const int dst = slot_dst[s0 + key];
            if (dst >= 0) w = *(const u32x4*)(dout + (int64_t)dst * channels + head * HD + half8 * 8);
        }
        return w;
    }, do_lds, dot_lds, t_stride);
    // a query that does not exist, or a filler slot, gets lse = +inf: its probabilities come out as zero
    for (int i = tid; i < len64; i += BWD_THREADS) {
        const bool real = i < len && slot_dst[s0 + i] >= 0;
        nlse_lds[i] = real ? -lse_ws[(int64_t)head * n_pad + s0 + i] : -INFINITY;
        nd_lds[i] = real ? -d_ws[(int64_t)head * n_pad + s0 + i] : 0.f;
    }
    __syncthreads();

    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int n_ktiles = (len + 31) / 32;
    const unsigned char* q_base = q_lds + col * 32 + hf * 16;
    const unsigned char* do_base = do_lds + col * 32 + hf * 16;
    const unsigned char* qt_base = col < HD ? qt_lds + (size_t)col * t_stride + hf * 32 : zero_lds;
    const unsigned char* dot_base = col < HD ? dot_lds + (size_t)col * t_stride + hf * 32 : zero_lds;
    const int t_step = col < HD ? 128 : 0;

    // Two key tiles per sweep over the queries: the query-side operands of a step (Q and dO rows, their
    // transposes, -lse and -D: 28 16-byte LDS reads) are fetched once and used for both, which halves the
    // LDS traffic per MFMA -- with one tile the kernel is bound by LDS bandwidth.
    const int kt_lo = (int)((int64_t)part * n_ktiles / parts), kt_hi = (int)((int64_t)(part + 1) * n_ktiles / parts);
    for (int kt = kt_lo + wave; kt < kt_hi; kt += 2 * BWD_WAVES) {
        int key[2], kdst[2];
        int64_t row[2];
        bool valid[2];
        v8 kfrag[2], vfrag[2];
        f32x16 acc_v[2], acc_k[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            key[t] = (kt + t * BWD_WAVES) * 32 + col;
            valid[t] = key[t] < len && kt + t * BWD_WAVES < kt_hi;
            row[t] = 0;
            kdst[t] = -1;
            u32x4 kreg = {0, 0, 0, 0}, vreg = {0, 0, 0, 0};
            if (valid[t]) {
                row[t] = slot_src[s0 + key[t]];
                kdst[t] = slot_dst[s0 + key[t]];
                kreg = *(const u32x4*)(qkv + row[t] * row_stride + channels + head * HD + hf * 8);
                vreg = *(const u32x4*)(qkv + row[t] * row_stride + 2 * channels + head * HD + hf * 8);
            }
            kfrag[t] = __builtin_bit_cast(v8, kreg);
            vfrag[t] = __builtin_bit_cast(v8, vreg);
            acc_v[t] = splat16(0.f);
            acc_k[t] = splat16(0.f);
        }
        const bool two = kt + BWD_WAVES < kt_hi;   // the same for every lane of the wave
        const unsigned char* qt_ptr = qt_base;
        const unsigned char* dot_ptr = dot_base;
        for (int st = 0; st < n_pairs; ++st) {
            const v8 q0 = __builtin_bit_cast(v8, *(const u32x4*)(q_base + (size_t)st * 64 * 32));
            const v8 q1 = __builtin_bit_cast(v8, *(const u32x4*)(q_base + (size_t)st * 64 * 32 + 32 * 32));
            const v8 g0 = __builtin_bit_cast(v8, *(const u32x4*)(do_base + (size_t)st * 64 * 32));
            const v8 g1 = __builtin_bit_cast(v8, *(const u32x4*)(do_base + (size_t)st * 64 * 32 + 32 * 32));
            // C operands: register v of a lane holds query 8 (v / 4) + 4 hf + v % 4 of the 32-block
            f32x16 cla, clb, cda, cdb;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int qa = st * 64 + 8 * a + 4 * hf;
                const f32x4 la = *(const f32x4*)(nlse_lds + qa), lb = *(const f32x4*)(nlse_lds + qa + 32);
                const f32x4 da = *(const f32x4*)(nd_lds + qa), db = *(const f32x4*)(nd_lds + qa + 32);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    cla[4 * a + r] = la[r];
                    clb[4 * a + r] = lb[r];
                    cda[4 * a + r] = da[r];
                    cdb[4 * a + r] = db[r];
                }
            }
            const v8 ga0 = __builtin_bit_cast(v8, *(const u32x4*)dot_ptr);
            const v8 ga1 = __builtin_bit_cast(v8, *(const u32x4*)(dot_ptr + 16));
            const v8 gb0 = __builtin_bit_cast(v8, *(const u32x4*)(dot_ptr + 64));
            const v8 gb1 = __builtin_bit_cast(v8, *(const u32x4*)(dot_ptr + 80));
            const v8 qa0 = __builtin_bit_cast(v8, *(const u32x4*)qt_ptr);
            const v8 qa1 = __builtin_bit_cast(v8, *(const u32x4*)(qt_ptr + 16));
            const v8 qb0 = __builtin_bit_cast(v8, *(const u32x4*)(qt_ptr + 64));
            const v8 qb1 = __builtin_bit_cast(v8, *(const u32x4*)(qt_ptr + 80));
            dot_ptr += t_step;
            qt_ptr += t_step;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                if (t == 1 && !two) break;
                const f32x16 zero = splat16(0.f);
                const f32x16 sa = Half<T>::mfma(q0, kfrag[t], cla);    // S - lse, [query, this lane's key]
                const f32x16 sb = Half<T>::mfma(q1, kfrag[t], clb);
                const f32x16 da = Half<T>::mfma(g0, vfrag[t], DROP ? zero : cda);    // dP - D (dP alone with dropout)
                const f32x16 db = Half<T>::mfma(g1, vfrag[t], DROP ? zero : cdb);
                float pa[16], pb[16], dsa[16], dsb[16];
                if (DROP) {
                    // the mask of (query, key): dV sees the kept, rescaled probabilities, dS = P o (mask o dP / (1 - p) - D)
                    const uint32_t hconst = (((uint32_t)head + 1u) * 0xC2B2AE3Du) ^ drop.seed;
                    const uint32_t kslot = (uint32_t)(s0 + key[t]);
                    const uint32_t q0s = (uint32_t)s0 + (uint32_t)st * 64u + 4u * (uint32_t)hf;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const uint32_t qs = q0s + 8u * (uint32_t)(v >> 2) + (uint32_t)(v & 3);
                        const bool ka = drop_keep((qs * 0x9E3779B1u) ^ hconst, kslot, drop.threshold);
                        const bool kb = drop_keep(((qs + 32u) * 0x9E3779B1u) ^ hconst, kslot, drop.threshold);
                        const float ea = __builtin_amdgcn_exp2f(sa[v]), eb = __builtin_amdgcn_exp2f(sb[v]);
                        pa[v] = ka ? ea * drop.inv_keep : 0.f;
                        pb[v] = kb ? eb * drop.inv_keep : 0.f;
                        dsa[v] = ea * ((ka ? da[v] * drop.inv_keep : 0.f) + cda[v]);   // cda holds -D
                        dsb[v] = eb * ((kb ? db[v] * drop.inv_keep : 0.f) + cdb[v]);
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        pa[v] = __builtin_amdgcn_exp2f(sa[v]);
                        pb[v] = __builtin_amdgcn_exp2f(sb[v]);
                        dsa[v] = pa[v] * da[v];
                        dsb[v] = pb[v] * db[v];
                    }
                }
                acc_v[t] = Half<T>::mfma(ga0, pack8<T>(pa), acc_v[t]);
                acc_v[t] = Half<T>::mfma(ga1, pack8<T>(pa + 8), acc_v[t]);
                acc_v[t] = Half<T>::mfma(gb0, pack8<T>(pb), acc_v[t]);
                acc_v[t] = Half<T>::mfma(gb1, pack8<T>(pb + 8), acc_v[t]);
                acc_k[t] = Half<T>::mfma(qa0, pack8<T>(dsa), acc_k[t]);
                acc_k[t] = Half<T>::mfma(qa1, pack8<T>(dsa + 8), acc_k[t]);
                acc_k[t] = Half<T>::mfma(qb0, pack8<T>(dsb), acc_k[t]);
                acc_k[t] = Half<T>::mfma(qb1, pack8<T>(dsb + 8), acc_k[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (!valid[t]) continue;
            // a real slot owns its row of dqkv; a filler's share is parked per slot and added afterwards.
            // Q^T was staged times scale * log2(e): dK = scale * dS^T Q = (dS^T Q_staged) * ln 2
            T* base = kdst[t] >= 0 ? dqkv + row[t] * row_stride + channels + head * HD + 4 * hf
                                   : fill + (int64_t)(s0 + key[t]) * 2 * channels + head * HD + 4 * hf;
            const f32x16 ak = acc_k[t], av = acc_v[t];
            u32x2 lo = {Half<T>::pack2(ak[0] * LN2, ak[1] * LN2), Half<T>::pack2(ak[2] * LN2, ak[3] * LN2)};
            u32x2 hi = {Half<T>::pack2(ak[4] * LN2, ak[5] * LN2), Half<T>::pack2(ak[6] * LN2, ak[7] * LN2)};
            *(u32x2*)base = lo;
            *(u32x2*)(base + 8) = hi;
            lo = (u32x2){Half<T>::pack2(av[0], av[1]), Half<T>::pack2(av[2], av[3])};
            hi = (u32x2){Half<T>::pack2(av[4], av[5]), Half<T>::pack2(av[6], av[7])};
            *(u32x2*)(base + channels) = lo;
            *(u32x2*)(base + channels + 8) = hi;
        }
    }
}

// ---- fp32: thread per query (kernel 1) and per key (kernel 2), 128-slot chunks in LDS
constexpr int F32_B = 256;    // queries / keys per block
constexpr int F32_C = 128;    // slots per chunk

// Relative position bias of model.py:297-316, :468-469 on the fp32 path: score(query i, key j, head h) +=
// sum over the axes a of table[a R + clamp(g_i[a] - g_j[a], -bnd, bnd) + bnd][h], R = 2 bnd + 1. grid == nullptr:
// no bias. dtable (3 R, heads) receives the table's gradient (sum of dS over the pairs that read an entry).
constexpr int RPE_MAX_BND = 128;
struct Rpe {
    const int32_t* grid;   // (n_rows, 3) grid coordinates in point order
    const float* table;    // (3 R, heads)
    float* dtable;         // (3 R, heads), accumulated into
    int bnd;
};
__device__ __forceinline__ int rpe_index(int q, int k, int bnd) { return min(max(q - k, -bnd), bnd) + bnd; }

__global__ __launch_bounds__(F32_B) void attn_bwd_q_f32_kernel(
    const float* __restrict__ qkv, const float* __restrict__ out, const float* __restrict__ dout, int channels,
    int heads, const int32_t* __restrict__ slot_src, const int32_t* __restrict__ slot_dst,
    const int32_t* __restrict__ cu_seqlens, int blocks, float scale, int64_t n_pad, float* __restrict__ dqkv,
    float* __restrict__ lse_ws, float* __restrict__ d_ws, Rpe rpe, Dropout drop) {
    __shared__ float k_lds[F32_C][HD];
    __shared__ float v_lds[F32_C][HD];
    __shared__ int32_t c_lds[F32_C][3];
    __shared__ float t_lds[3 * (2 * RPE_MAX_BND + 1)], dt_lds[3 * (2 * RPE_MAX_BND + 1)];
    const int seq = blockIdx.x / (heads * blocks);
    const int rem = blockIdx.x % (heads * blocks);
    const int head = rem / blocks, qb = rem % blocks;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (qb * F32_B >= len) return;
    const int tid = threadIdx.x;
    const int qi = qb * F32_B + tid;
    const int64_t row_stride = 3 * (int64_t)channels;
    const int rnum = 2 * rpe.bnd + 1;
    if (rpe.grid) {
        for (int e = tid; e < 3 * rnum; e += F32_B) {
            t_lds[e] = rpe.table[(int64_t)e * heads + head];
            dt_lds[e] = 0.f;
        }
    }

    float q[HD], g[HD], dq[HD];
    int dst = -1, qx = 0, qy = 0, qz = 0;
    float dsum = 0.f;
#pragma unroll
    for (int d = 0; d < HD; ++d) { q[d] = 0.f; g[d] = 0.f; dq[d] = 0.f; }
    if (qi < len) dst = slot_dst[s0 + qi];
    if (dst >= 0 && rpe.grid) {
        qx = rpe.grid[3 * (int64_t)dst];
        qy = rpe.grid[3 * (int64_t)dst + 1];
        qz = rpe.grid[3 * (int64_t)dst + 2];
    }
    if (dst >= 0) {
        const float* src = qkv + (int64_t)dst * row_stride + head * HD;
        const float* gs = dout + (int64_t)dst * channels + head * HD;
        const float* os = out + (int64_t)dst * channels + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) {
            q[d] = src[d] * scale;
            g[d] = gs[d];
            dsum = fmaf(g[d], os[d], dsum);
        }
    }
    float m = -INFINITY, l = 0.f, lse = 0.f;
    const uint32_t hq = drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + qi));
    for (int sweep = 0; sweep < 2; ++sweep) {
        for (int c0 = 0; c0 < len; c0 += F32_C) {
            __syncthreads();
            for (int e = tid; e < F32_C * HD; e += F32_B) {
                const int key = e / HD, d = e % HD;
                float kv = 0.f, vv = 0.f;
                if (c0 + key < len) {
                    const int64_t r = slot_src[s0 + c0 + key];
                    const float* src = qkv + r * row_stride + head * HD + d;
                    kv = src[channels];
                    vv = src[2 * channels];
                    if (rpe.grid && d < 3) c_lds[key][d] = rpe.grid[3 * r + d];
                }
                k_lds[key][d] = kv;
                v_lds[key][d] = vv;
            }
            __syncthreads();
            const int kn = min(F32_C, len - c0);
            for (int key = 0; key < kn; ++key) {
                float s = 0.f;
#pragma unroll
                for (int d = 0; d < HD; ++d) s = fmaf(q[d], k_lds[key][d], s);
                int bx = 0, by = 0, bz = 0;
                if (rpe.grid) {
                    bx = rpe_index(qx, c_lds[key][0], rpe.bnd);
                    by = rnum + rpe_index(qy, c_lds[key][1], rpe.bnd);
                    bz = 2 * rnum + rpe_index(qz, c_lds[key][2], rpe.bnd);
                    s += t_lds[bx] + t_lds[by] + t_lds[bz];
                }
                if (sweep == 0) {
                    if (s > m) {
                        l *= __expf(m - s);
                        m = s;
                    }
                    l += __expf(s - m);
                } else {
                    const float p = __expf(s - lse);
                    float dp = 0.f;
#pragma unroll
                    for (int d = 0; d < HD; ++d) dp = fmaf(g[d], v_lds[key][d], dp);
                    if (drop.threshold)
                        dp = drop_keep(hq, (uint32_t)(s0 + c0 + key), drop.threshold) ? dp * drop.inv_keep : 0.f;
                    const float ds = p * (dp - dsum);
#pragma unroll
                    for (int d = 0; d < HD; ++d) dq[d] = fmaf(ds, k_lds[key][d], dq[d]);
                    if (rpe.grid && dst >= 0) {   // every (query, key) pair is seen exactly once, here
                        atomicAdd(&dt_lds[bx], ds);
                        atomicAdd(&dt_lds[by], ds);
                        atomicAdd(&dt_lds[bz], ds);
                    }
                }
            }
        }
        if (sweep == 0) lse = m + __logf(l);
    }
    if (dst >= 0) {
        float* o = dqkv + (int64_t)dst * row_stride + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) o[d] = dq[d] * scale;
        lse_ws[(int64_t)head * n_pad + s0 + qi] = lse;   // natural-log units on this path
        d_ws[(int64_t)head * n_pad + s0 + qi] = dsum;
    }
    if (rpe.grid) {
        __syncthreads();
        for (int e = tid; e < 3 * rnum; e += F32_B)
            if (dt_lds[e] != 0.f) atomicAdd(rpe.dtable + (int64_t)e * heads + head, dt_lds[e]);
    }
}

__global__ __launch_bounds__(F32_B) void attn_bwd_kv_f32_kernel(
    const float* __restrict__ qkv, const float* __restrict__ dout, int channels, int heads,
    const int32_t* __restrict__ slot_src, const int32_t* __restrict__ slot_dst,
    const int32_t* __restrict__ cu_seqlens, int blocks, float scale, int64_t n_pad,
    const float* __restrict__ lse_ws, const float* __restrict__ d_ws, float* __restrict__ dqkv,
    float* __restrict__ fill, Rpe rpe, Dropout drop) {
    __shared__ float q_lds[F32_C][HD];    // q * scale
    __shared__ float g_lds[F32_C][HD];    // dO
    __shared__ float lse_lds[F32_C];
    __shared__ float d_lds[F32_C];
    __shared__ int32_t c_lds[F32_C][3];
    __shared__ float t_lds[3 * (2 * RPE_MAX_BND + 1)];
    const int seq = blockIdx.x / (heads * blocks);
    const int rem = blockIdx.x % (heads * blocks);
    const int head = rem / blocks, kb = rem % blocks;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (kb * F32_B >= len) return;
    const int tid = threadIdx.x;
    const int ki = kb * F32_B + tid;
    const int64_t row_stride = 3 * (int64_t)channels;

    const int rnum = 2 * rpe.bnd + 1;
    if (rpe.grid)
        for (int e = tid; e < 3 * rnum; e += F32_B) t_lds[e] = rpe.table[(int64_t)e * heads + head];
    float k[HD], v[HD], dk[HD], dv[HD];
    int64_t row = 0;
    int kx = 0, ky = 0, kz = 0;
#pragma unroll
    for (int d = 0; d < HD; ++d) { k[d] = 0.f; v[d] = 0.f; dk[d] = 0.f; dv[d] = 0.f; }
    if (ki < len && rpe.grid) {
        const int64_t r = slot_src[s0 + ki];
        kx = rpe.grid[3 * r];
        ky = rpe.grid[3 * r + 1];
        kz = rpe.grid[3 * r + 2];
    }
    if (ki < len) {
        row = slot_src[s0 + ki];
        const float* src = qkv + row * row_stride + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) {
            k[d] = src[channels + d];
            v[d] = src[2 * channels + d];
        }
    }
    for (int c0 = 0; c0 < len; c0 += F32_C) {
        __syncthreads();
        for (int e = tid; e < F32_C * HD; e += F32_B) {
            const int qi = e / HD, d = e % HD;
            float qv = 0.f, gv = 0.f;
            if (c0 + qi < len) {
                const int dst = slot_dst[s0 + c0 + qi];
                if (dst >= 0) {
                    qv = qkv[(int64_t)dst * row_stride + head * HD + d] * scale;
                    gv = dout[(int64_t)dst * channels + head * HD + d];
                    if (rpe.grid && d < 3) c_lds[qi][d] = rpe.grid[3 * (int64_t)dst + d];
                }
            }
            q_lds[qi][d] = qv;
            g_lds[qi][d] = gv;
        }
        if (tid < F32_C) {
            const bool real = c0 + tid < len && slot_dst[s0 + c0 + tid] >= 0;
            lse_lds[tid] = real ? lse_ws[(int64_t)head * n_pad + s0 + c0 + tid] : INFINITY;
            d_lds[tid] = real ? d_ws[(int64_t)head * n_pad + s0 + c0 + tid] : 0.f;
        }
        __syncthreads();
        const int qn = min(F32_C, len - c0);
        for (int qi = 0; qi < qn; ++qi) {
            float s = 0.f, dp = 0.f;
#pragma unroll
            for (int d = 0; d < HD; ++d) {
                s = fmaf(q_lds[qi][d], k[d], s);
                dp = fmaf(g_lds[qi][d], v[d], dp);
            }
            if (rpe.grid && lse_lds[qi] != INFINITY)   // a real query: its coordinates are in c_lds
                s += t_lds[rpe_index(c_lds[qi][0], kx, rpe.bnd)] + t_lds[rnum + rpe_index(c_lds[qi][1], ky, rpe.bnd)] +
                     t_lds[2 * rnum + rpe_index(c_lds[qi][2], kz, rpe.bnd)];
            const float p = __expf(s - lse_lds[qi]);
            float pv = p;   // what multiplied V in the forward pass
            if (drop.threshold) {
                const bool keep = drop_keep(drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + c0 + qi)), (uint32_t)(s0 + ki),
                                            drop.threshold);
                pv = keep ? p * drop.inv_keep : 0.f;
                dp = keep ? dp * drop.inv_keep : 0.f;
            }
            const float ds = p * (dp - d_lds[qi]);
#pragma unroll
            for (int d = 0; d < HD; ++d) {
                dv[d] = fmaf(pv, g_lds[qi][d], dv[d]);
                dk[d] = fmaf(ds, q_lds[qi][d], dk[d]);   // q already carries the scale
            }
        }
    }
    if (ki < len) {
        float* base = slot_dst[s0 + ki] >= 0 ? dqkv + row * row_stride + channels + head * HD
                                             : fill + (int64_t)(s0 + ki) * 2 * channels + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) {
            base[d] = dk[d];
            base[channels + d] = dv[d];
        }
    }
}

// Filler slots: their dK and dV, parked per slot, are added to the row the slot repeats. A row is
// repeated by at most one filler slot, so plain read-modify-write is race-free.
template <typename T>
__global__ __launch_bounds__(256) void attn_bwd_fill_kernel(const T* __restrict__ fill, int channels,
                                                            const int32_t* __restrict__ slot_src,
                                                            const int32_t* __restrict__ slot_dst, int64_t n_pad,
                                                            T* __restrict__ dqkv) {
    const int per = 2 * channels / 8;   // 8-channel pieces per slot
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_pad * per) return;
    const int64_t slot = i / per;
    const int piece = (int)(i % per);
    if (slot_dst[slot] >= 0) return;
    const T* src = fill + slot * 2 * channels + piece * 8;
    T* dst = dqkv + (int64_t)slot_src[slot] * 3 * channels + channels + piece * 8;
#pragma unroll
    for (int c = 0; c < 8; ++c) dst[c] = (T)((float)dst[c] + (float)src[c]);
}

struct BwdWs {
    float* lse;
    float* d;
    void* fill;
    size_t bytes;
};

BwdWs carve(void* base, int dtype, int64_t n_pad, int channels, int heads) {
    const size_t elt = dtype == PTV3_F32 ? 4 : 2;
    BwdWs w;
    size_t off = 0;
    w.lse = (float*)((char*)base + off);
    off += ptv3_align256((size_t)n_pad * heads * sizeof(float));
    w.d = (float*)((char*)base + off);
    off += ptv3_align256((size_t)n_pad * heads * sizeof(float));
    w.fill = (char*)base + off;
    off += ptv3_align256((size_t)n_pad * 2 * channels * elt);
    w.bytes = off;
    return w;
}

template <typename T>
int launch_half_bwd(const void* qkv, const void* out, const void* dout, int channels, int heads,
                    const int32_t* slot_src, const int32_t* slot_dst, const int32_t* cu_seqlens, int64_t n_seq,
                    int64_t max_seqlen, int64_t n_pad, float scale, void* dqkv, const BwdWs& ws, float* lse, Dropout drop,
                    hipStream_t stream) {
    const int lds_keys = (int)((max_seqlen + 63) & ~63ll);
    const size_t t_bytes = (size_t)HD * (lds_keys * 2 + VT_PAD_BYTES);
    const size_t lds_q = 2 * (size_t)lds_keys * 32 + t_bytes + 96;
    const size_t lds_kv = 2 * (size_t)lds_keys * 32 + 2 * t_bytes + 2 * (size_t)lds_keys * sizeof(float) + 96;
    if (lds_q > 160 * 1024 || lds_kv > 160 * 1024) return PTV3_ESHAPE;
    const bool dropping = drop.threshold != 0u;
    auto kq = dropping ? (lse ? attn_bwd_q_kernel<T, true, true> : attn_bwd_q_kernel<T, false, true>)
                       : (lse ? attn_bwd_q_kernel<T, true, false> : attn_bwd_q_kernel<T, false, false>);
    float* lse_buf = lse ? lse : ws.lse;
    auto kkv = dropping ? attn_bwd_kv_kernel<T, true> : attn_bwd_kv_kernel<T, false>;
    static LdsGrant grant_q[4], grant_kv[2];   // per kernel variant and device
    const int qi_ = (lse != nullptr) + 2 * dropping;
    if (const int rc_ = ptv3_allow_lds((const void*)kq, lds_q, grant_q[qi_])) return rc_;
    if (const int rc_ = ptv3_allow_lds((const void*)kkv, lds_kv, grant_kv[dropping])) return rc_;
    // one work-group per CU is resident (LDS): the items beyond the last full round are cut into ranges of
    // tiles when that shortens the round (each range stages the sequence again, about 0.15 of an item)
    static int slots = 0;
    if (slots == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        slots = cus;
    }
    const int64_t total = n_seq * heads;
    const int64_t rem = total % slots;
    int64_t full = total - rem, split = 1;
    if (rem != 0) {
        double best = 1.0;
        for (int64_t sp = 2; sp <= 4; ++sp) {
            const double cost = (double)((rem * sp + slots - 1) / slots) * (1.0 / (double)sp + 0.15);
            if (cost < best - 1e-9) { best = cost; split = sp; }
        }
    }
    if (split == 1) full = total;
    const unsigned grid = (unsigned)(full + (total - full) * split);
    hipLaunchKernelGGL(kq, dim3(grid), dim3(BWQ_THREADS), lds_q, stream, (const T*)qkv, (const T*)out, (const T*)dout,
                       channels, heads, slot_src, slot_dst, cu_seqlens, lds_keys, scale, n_pad, (T*)dqkv, lse_buf, ws.d,
                       (int)full, (int)split, drop);
    hipLaunchKernelGGL(kkv, dim3(grid), dim3(BWD_THREADS), lds_kv, stream, (const T*)qkv, (const T*)dout, channels,
                       heads, slot_src, slot_dst, cu_seqlens, lds_keys, scale, n_pad, lse_buf, ws.d, (T*)dqkv,
                       (T*)ws.fill, (int)full, (int)split, drop);
    const int64_t items = n_pad * (2 * channels / 8);
    hipLaunchKernelGGL(attn_bwd_fill_kernel<T>, dim3((unsigned)ptv3_ceil_div(items, 256)), dim3(256), 0, stream,
                       (const T*)ws.fill, channels, slot_src, slot_dst, n_pad, (T*)dqkv);
    PTV3_RETURN_LAUNCH();
}

}  // namespace

extern "C" size_t ptv3_patch_attn_bwd_workspace_bytes(int dtype, int64_t n_pad, int channels, int heads) {
    if (n_pad < 0 || channels < 1 || heads < 1) return 0;
    return carve(nullptr, dtype, n_pad, channels, heads).bytes;
}

extern "C" int ptv3_patch_attn_bwd(const void* qkv, const void* out, const void* dout, int dtype, int64_t n_rows,
                                   int channels, int heads, const int32_t* slot_src, const int32_t* slot_dst,
                                   const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen, int64_t n_pad,
                                   float scale, const float* lse, float dropout_p, uint32_t dropout_seed, void* dqkv,
                                   void* workspace, size_t workspace_bytes, void* stream_) {
    return ptv3_patch_attn_rpe_bwd(qkv, out, dout, dtype, n_rows, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                   max_seqlen, n_pad, scale, lse, dropout_p, dropout_seed, nullptr, nullptr, 0, nullptr,
                                   dqkv, workspace, workspace_bytes, stream_);
}

extern "C" int ptv3_patch_attn_rpe_bwd(const void* qkv, const void* out, const void* dout, int dtype, int64_t n_rows,
                                       int channels, int heads, const int32_t* slot_src, const int32_t* slot_dst,
                                       const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen, int64_t n_pad,
                                       float scale, const float* lse, float dropout_p, uint32_t dropout_seed,
                                       const int32_t* grid_coord, const float* rpe_table, int pos_bnd,
                                       float* drpe_table, void* dqkv, void* workspace, size_t workspace_bytes,
                                       void* stream_) {
    if (grid_coord && (dtype != PTV3_F32 || !rpe_table || !drpe_table)) return PTV3_ESHAPE;   // the bias lives on the fp32 path
    if (grid_coord && (pos_bnd < 0 || pos_bnd > RPE_MAX_BND)) return PTV3_ESHAPE;
    if (!(dropout_p >= 0.f) || !(dropout_p < 1.f)) return PTV3_EINVAL;
    const Rpe rpe = {grid_coord, rpe_table, drpe_table, grid_coord ? pos_bnd : 0};
    const Dropout drop = {dropout_seed, dropout_p > 0.f ? drop_threshold(dropout_p) : 0u, 1.f / (1.f - dropout_p)};
    if (n_rows < 0 || n_seq < 0 || n_pad < 0 || channels < 1 || heads < 1 || max_seqlen < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (channels % heads != 0 || channels / heads != HD) return PTV3_ESHAPE;
    if (n_seq * heads >= (1ll << 31)) return PTV3_EINVAL;
    if (n_seq == 0 || n_rows == 0 || n_pad == 0) return PTV3_OK;
    if (!qkv || !out || !dout || !slot_src || !slot_dst || !cu_seqlens || !dqkv || !workspace) return PTV3_EINVAL;
    const BwdWs ws = carve(workspace, dtype, n_pad, channels, heads);
    if (workspace_bytes < ws.bytes) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16)
        return launch_half_bwd<_Float16>(qkv, out, dout, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                         max_seqlen, n_pad, scale, dqkv, ws, (float*)lse, drop, stream);
    if (dtype == PTV3_BF16)
        return launch_half_bwd<__bf16>(qkv, out, dout, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                       max_seqlen, n_pad, scale, dqkv, ws, (float*)lse, drop, stream);
    const int blocks = (int)ptv3_ceil_div(max_seqlen, F32_B);
    if (n_seq * heads * blocks >= (1ll << 31)) return PTV3_EINVAL;
    const unsigned grid = (unsigned)(n_seq * heads * blocks);
    hipLaunchKernelGGL(attn_bwd_q_f32_kernel, dim3(grid), dim3(F32_B), 0, stream, (const float*)qkv, (const float*)out,
                       (const float*)dout, channels, heads, slot_src, slot_dst, cu_seqlens, blocks, scale, n_pad,
                       (float*)dqkv, ws.lse, ws.d, rpe, drop);
    hipLaunchKernelGGL(attn_bwd_kv_f32_kernel, dim3(grid), dim3(F32_B), 0, stream, (const float*)qkv,
                       (const float*)dout, channels, heads, slot_src, slot_dst, cu_seqlens, blocks, scale, n_pad, ws.lse,
                       ws.d, (float*)dqkv, (float*)ws.fill, rpe, drop);
    const int64_t items = n_pad * (2 * channels / 8);
    hipLaunchKernelGGL(attn_bwd_fill_kernel<float>, dim3((unsigned)ptv3_ceil_div(items, 256)), dim3(256), 0, stream,
                       (const float*)ws.fill, channels, slot_src, slot_dst, n_pad, (float*)dqkv);
    PTV3_RETURN_LAUNCH();
}
