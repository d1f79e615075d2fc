// Serialized patch attention, head_dim 16, fused with the gathers either side of it.
//
// Replaces model.py:456-484 of the reference (row gather qkv[order], the
// flash_attn_varlen_qkvpacked_func call / torch fallback, row gather feat[inverse]).
//
// Half-precision kernel (fp16 / bf16), one workgroup per (sequence, head):
//   * K (row-major) and V (transposed, key axis permuted to the MFMA register order) of the
//     whole sequence sit in LDS: 2 * 1024 * 16 * 2 B = 64 KB for a 1024-point patch, so K/V
//     are fetched from HBM exactly once per (sequence, head).
//   * Scores are produced transposed, S^T = K * Q^T, with v_mfma_f32_32x32x16: the
//     contraction length 16 is exactly one head, and in the result every lane owns ONE
//     query (column) and 16 keys (rows). Row max / rescale are then lane-local apart from a
//     single exchange with lane^32, and the fp32 result registers, converted to 16-bit,
//     are already in operand layout for the second product O^T = V^T * P^T.
//   * V^T only fills 16 of the 32 rows of that product; rows 16 and 20 are fed ones (from a small
//     LDS constant, by per-lane addressing) so the softmax denominator falls out of the same MFMA
//     instead of costing VALU adds.
//   * At head_dim 16 the kernel is bound by the softmax arithmetic, not by the MFMAs: per 64 keys x
//     32 queries a wave issues 6 MFMAs (128 useful MFMA cycles) but 32 v_exp_f32 (8 issue cycles
//     each on this part) and 16 packed conversions (4 each), 320 VALU cycles. Everything else is
//     therefore taken off the VALU: q is scaled by scale*log2(e) once; a |q||k| bound (key norms are
//     reduced while K is staged) decides per query tile whether probabilities can be taken as
//     2^score with no running maximum at all (C operand = constant zero); otherwise the running
//     reference maximum enters through the MFMA's C operand so scores arrive already shifted, and
//     the reference only moves when a score exceeds it by 2^8 -- which the same bound rules out
//     for most 64-key steps without looking at the scores.
//   * Rows are read through slot_src and written through slot_dst, so the padded,
//     permuted qkv tensor of the reference is never materialised.
// fp32 kernel: one thread per query, K/V chunks staged in LDS, plain FMA arithmetic.
#include "attn_half.h"

namespace {

// Scores may exceed the running reference maximum by this much (log2 units) before the
// accumulators are rescaled: probabilities then stay below 2^8, safe for fp16 operands.
constexpr float RESCALE_SLACK = 8.f;

// One 32-query tile of one wave against every key of the sequence in LDS.
// SHIFT = false: the caller has checked that no score can leave [-limit, limit] (|q||k| bound),
// so probabilities 2^score are representable as they are, the MFMA's C operand is the constant
// zero and the loop holds nothing but loads, MFMAs, exponentials and conversions.
// SHIFT = true: scores arrive shifted by a running reference maximum that enters through the C
// operand; the reference moves (and the accumulators are rescaled) only when a score exceeds it
// by RESCALE_SLACK, which the per-step |q||k| bound rules out without looking at the scores.
// DROP: attention dropout. The denominator is then summed on the VALU from the probabilities before the mask
// (the ones row of the second product would add up the masked ones) and handed back in acc[8] like the other.
template <typename T, bool SHIFT, bool LSE, bool DROP>
__device__ __forceinline__ f32x16 attend_tile(typename Half<T>::v8 qfrag, float qnorm, float kn_reg,
                                              const unsigned char* k_ptr, const unsigned char* v_ptr,
                                              int v_step, int n_pairs, int len, int hf, Dropout drop, uint32_t hq,
                                              uint32_t kslot0) {
    typedef typename Half<T>::v8 v8;
    f32x16 acc, cinit;
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc[v] = 0.f; cinit[v] = 0.f; }
    float m_ref = 0.f;   // reference maximum: the MFMA adds -m_ref to every score
    float den = 0.f;     // DROP: sum of the probabilities this lane has seen
    const bool ragged = (len & 63) != 0;
    v8 k0 = __builtin_bit_cast(v8, *(const u32x4*)k_ptr);
    v8 k1 = __builtin_bit_cast(v8, *(const u32x4*)(k_ptr + 32 * 32));
    for (int kp = 0; kp < n_pairs; ++kp) {
        f32x16 sa = Half<T>::mfma(k0, qfrag, cinit);   // sa[v] = <K[key_v], Q[q]> - m_ref
        f32x16 sb = Half<T>::mfma(k1, qfrag, cinit);
        // operands of the second product: 16 value rows, a row of ones (the denominator), zeros
        const u32x4 va0 = *(const u32x4*)v_ptr;
        const u32x4 va1 = *(const u32x4*)(v_ptr + 16);
        const u32x4 vb0 = *(const u32x4*)(v_ptr + 64);
        const u32x4 vb1 = *(const u32x4*)(v_ptr + 80);
        v_ptr += v_step;
        // keys of the next step (the tile is padded by one step, so the address is always valid)
        k_ptr += 64 * 32;
        k0 = __builtin_bit_cast(v8, *(const u32x4*)k_ptr);
        k1 = __builtin_bit_cast(v8, *(const u32x4*)(k_ptr + 32 * 32));
        if (ragged && kp == n_pairs - 1) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int key = kp * 64 + 8 * (v >> 2) + 4 * hf + (v & 3);
                if (key >= len) sa[v] = -INFINITY;
                if (key + 32 >= len) sb[v] = -INFINITY;
            }
        }
        if (SHIFT) {
            // |score| <= |q| |k|: when even that bound stays within the slack nothing can
            // overflow and the running reference is left alone (no max reduction at all)
            const float kn = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kn_reg), kp));
            const bool first = (kp == 0);
            if (first || __ballot(qnorm * kn - m_ref > RESCALE_SLACK) != 0) {
                float mx = fmaxf(sa[0], sb[0]);
#pragma unroll
                for (int v = 1; v < 16; ++v) mx = fmaxf(mx, fmaxf(sa[v], sb[v]));
                mx = fmaxf(mx, __shfl_xor(mx, 32, PTV3_WAVE));
                const bool move = first || mx > RESCALE_SLACK;
                if (__ballot(move) != 0) {
                    const float delta = move ? mx : 0.f;
                    const float alpha = first ? 1.f : exp2f(-delta);
                    m_ref += delta;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        sa[v] -= delta;
                        sb[v] -= delta;
                        cinit[v] = -m_ref;
                    }
#pragma unroll
                    for (int v = 0; v < 9; ++v) acc[v] *= alpha;   // rows 0..15 + denominator row
                    if (DROP) den *= alpha;
                }
            }
        }
        uint32_t pa[8], pb[8];
        if (DROP) {
            const uint32_t k0s = kslot0 + (uint32_t)kp * 64u + 4u * (uint32_t)hf;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                float e[4] = {__builtin_amdgcn_exp2f(sa[2 * v]), __builtin_amdgcn_exp2f(sa[2 * v + 1]),
                              __builtin_amdgcn_exp2f(sb[2 * v]), __builtin_amdgcn_exp2f(sb[2 * v + 1])};
                den += (e[0] + e[1]) + (e[2] + e[3]);
                // register i of the first 32-block holds key 8 (i / 4) + 4 hf + i % 4; the second block is 32 on
                const uint32_t ka = k0s + 8u * (uint32_t)((2 * v) >> 2) + (uint32_t)((2 * v) & 3);
                if (!drop_keep(hq, ka, drop.threshold)) e[0] = 0.f;
                if (!drop_keep(hq, ka + 1u, drop.threshold)) e[1] = 0.f;
                if (!drop_keep(hq, ka + 32u, drop.threshold)) e[2] = 0.f;
                if (!drop_keep(hq, ka + 33u, drop.threshold)) e[3] = 0.f;
                pa[v] = Half<T>::pack2(e[0], e[1]);
                pb[v] = Half<T>::pack2(e[2], e[3]);
            }
        } else {
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                pa[v] = Half<T>::pack2(__builtin_amdgcn_exp2f(sa[2 * v]), __builtin_amdgcn_exp2f(sa[2 * v + 1]));
                pb[v] = Half<T>::pack2(__builtin_amdgcn_exp2f(sb[2 * v]), __builtin_amdgcn_exp2f(sb[2 * v + 1]));
            }
        }
        acc = Half<T>::mfma(__builtin_bit_cast(v8, va0), __builtin_bit_cast(v8, (u32x4){pa[0], pa[1], pa[2], pa[3]}), acc);
        acc = Half<T>::mfma(__builtin_bit_cast(v8, va1), __builtin_bit_cast(v8, (u32x4){pa[4], pa[5], pa[6], pa[7]}), acc);
        acc = Half<T>::mfma(__builtin_bit_cast(v8, vb0), __builtin_bit_cast(v8, (u32x4){pb[0], pb[1], pb[2], pb[3]}), acc);
        acc = Half<T>::mfma(__builtin_bit_cast(v8, vb1), __builtin_bit_cast(v8, (u32x4){pb[4], pb[5], pb[6], pb[7]}), acc);
    }
    // result row 17 / 21 multiplies zeros: its register carries the reference maximum to the caller
    if (SHIFT && LSE) acc[9] = m_ref;
    if (DROP) acc[8] = den + __shfl_xor(den, 32, PTV3_WAVE);   // the other half-wave saw the other keys
    return acc;
}

// LSE: also write log2(sum_j 2^score_ij) of every real query, scores in log2 units (scale * log2(e) folded into
// q), to lse[head * lse_stride + slot]: what the backward kernels need to rebuild the probabilities.
template <typename T, bool LSE, bool DROP>
__global__ __launch_bounds__(ATT_THREADS, 4) void patch_attn_half_kernel(
    const T* __restrict__ qkv, int channels, int heads, const int32_t* __restrict__ slot_src,
    const int32_t* __restrict__ slot_dst, const int32_t* __restrict__ cu_seqlens, int lds_keys,
    float scale_log2e, T* __restrict__ out, int full_items, int split, int total_items, float* __restrict__ lse,
    int64_t lse_stride, Dropout drop) {
    typedef typename Half<T>::v8 v8;
    extern __shared__ __align__(16) unsigned char smem[];
    // K tile: lds_keys + 64 rows of 32 B (the last 64 are only ever prefetched). V^T tile: 16 rows
    // of (lds_keys*2 + pad) B. One float per 64-key step: the largest squared key norm of the
    // step. Then 96 B of ones and 96 B of zeros: rows 16.. of the second product's A operand.
    unsigned char* k_lds = smem;
    const int vt_stride = lds_keys * 2 + VT_PAD_BYTES;
    unsigned char* vt_lds = smem + (size_t)(lds_keys + 64) * 32;
    float* knorm_lds = (float*)(vt_lds + (size_t)HD * vt_stride);
    unsigned char* const_lds = (unsigned char*)knorm_lds + ((lds_keys / 64 * 4 + 15) & ~15);

    // The first `full_items` work-groups take one (sequence, head) each. The items left over
    // after the last full round of resident work-groups are cut into `split` query ranges, one
    // work-group each, so that the partial round at the end of the launch is short.
    int wg, part = 0, parts = 1;
    if ((int)blockIdx.x < full_items) {
        wg = xcd_chunked_id(blockIdx.x, full_items);
    } else {
        // Work-group ids go round the XCDs (full_items is a multiple of the resident work-groups). Every XCD takes a
        // contiguous eighth of the tail's items, range after range of one item, then the next item: the ranges of
        // an item meet in one L2 (the keys and values the later ranges stage are there), and so do the heads of a
        // sequence, which read neighbouring pieces of the same cache lines.
        const int r = blockIdx.x - full_items;
        const int xcd = r & 7, j = r >> 3;
        const int per = (total_items - full_items + 7) >> 3;
        wg = full_items + xcd * per + j / split;
        part = j % split;
        parts = split;
        if (j / split >= per || wg >= total_items) return;
    }
    const int seq = wg / heads, head = wg % heads;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (len <= 0) return;
    const int len64 = (len + 63) & ~63;
    const int n_pairs = len64 / 64;
    const int tid = threadIdx.x;
    const int64_t row_stride = 3 * (int64_t)channels;

    for (int i = tid; i < n_pairs; i += ATT_THREADS) knorm_lds[i] = 0.f;
    if (tid < 48) ((uint32_t*)const_lds)[tid] = tid < 24 ? Half<T>::one() * 0x10001u : 0u;
    __syncthreads();
    // ---- stage K and V^T: a thread handles (key, 8-channel half); four items in flight per thread
    for (int e0 = tid; e0 < len64 * 2; e0 += 4 * ATT_THREADS) {
        int32_t row[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int key = (e0 + j * ATT_THREADS) >> 1;
            row[j] = key < len ? slot_src[s0 + key] : -1;
        }
        u32x4 kq[4], vq[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            kq[j] = (u32x4){0, 0, 0, 0};
            vq[j] = (u32x4){0, 0, 0, 0};
            if (row[j] >= 0) {
                const T* base = qkv + (int64_t)row[j] * row_stride + head * HD + (tid & 1) * 8;
                kq[j] = *(const u32x4*)(base + channels);
                vq[j] = *(const u32x4*)(base + 2 * channels);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = e0 + j * ATT_THREADS;
            if (e >= len64 * 2) break;
            const int key = e >> 1, half8 = e & 1;   // == tid & 1: the stride is even
            *(u32x4*)(k_lds + key * 32 + half8 * 16) = kq[j];
            float nsq = sum_sq8<T>(kq[j]);
            nsq += __shfl_xor(nsq, 1, PTV3_WAVE);   // the other half of the same key
            if (half8 == 0) atomicMax((int*)&knorm_lds[key >> 6], __float_as_int(nsq));   // nsq >= 0
            const int pos = (key & ~31) + vt_pos(key & 31);
            unsigned char* vt = vt_lds + (size_t)(half8 * 8) * vt_stride + pos * 2;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t w = vq[j][c];
                *(uint16_t*)(vt + (size_t)(2 * c) * vt_stride) = (uint16_t)(w & 0xffffu);
                *(uint16_t*)(vt + (size_t)(2 * c + 1) * vt_stride) = (uint16_t)(w >> 16);
            }
        }
    }
    __syncthreads();

    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int n_qtiles = (len + 31) / 32;

    // lane l keeps the largest key norm of step l (at most 37 steps fit the LDS); the largest of all
    float kn_reg = lane < n_pairs ? sqrtf(knorm_lds[lane]) * 1.0009765625f : 0.f;   // margin for rounding in the bound
    float kn_all = kn_reg;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) kn_all = fmaxf(kn_all, __shfl_xor(kn_all, off, PTV3_WAVE));

    // A operand rows of the second product: d < 16 read V^T and advance 128 B per step; rows 16
    // and 20 read ones and the others zeros, without advancing.
    const unsigned char* k_base = k_lds + col * 32 + hf * 16;
    const unsigned char* v_base = col < HD ? vt_lds + (size_t)col * vt_stride + hf * 32
                                           : const_lds + ((col == 16 || col == 20) ? 0 : 96);
    const int v_step = col < HD ? 128 : 0;

    const int qt_lo = (int)((int64_t)part * n_qtiles / parts), qt_hi = (int)((int64_t)(part + 1) * n_qtiles / parts);
    for (int qt = qt_lo + wave; qt < qt_hi; qt += ATT_WAVES) {
        const int qi = qt * 32 + col;   // my query inside the sequence
        int dst = -1;
        u32x4 qreg = {0, 0, 0, 0};
        if (qi < len) {
            dst = slot_dst[s0 + qi];
            qreg = *(const u32x4*)(qkv + (int64_t)slot_src[s0 + qi] * row_stride + head * HD + hf * 8);
        }
        if (__ballot(dst >= 0) == 0) continue;   // tile of filler slots only
        // scores come out of the MFMA in log2 units: q is scaled by scale * log2(e) up front
        qreg = scale8<T>(qreg, scale_log2e);
        const v8 qfrag = __builtin_bit_cast(v8, qreg);
        float qn = sum_sq8<T>(qreg);
        qn += __shfl_xor(qn, 32, PTV3_WAVE);
        // the hardware square root (one instruction, within an ulp) under the same margin: this is a bound, and the
        // correctly rounded one is twenty instructions for every tile of 32 queries
        const float qnorm = __builtin_amdgcn_sqrtf(qn) * 1.0009765625f;

        f32x16 acc;
        const uint32_t hq = DROP ? drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + qi)) : 0u;
        if (__ballot(qnorm * kn_all > Half<T>::plain_limit()) == 0)
            acc = attend_tile<T, false, LSE, DROP>(qfrag, qnorm, kn_reg, k_base, v_base, v_step, n_pairs, len, hf, drop, hq,
                                                   (uint32_t)s0);
        else
            acc = attend_tile<T, true, LSE, DROP>(qfrag, qnorm, kn_reg, k_base, v_base, v_step, n_pairs, len, hf, drop, hq,
                                                  (uint32_t)s0);
        // acc[v]: d = 8*(v/4) + 4*hf + v%4; acc[8] = sum of probabilities (row 16 / 20)
        if (dst >= 0) {
            const float inv = (DROP ? drop.inv_keep : 1.f) / acc[8];
            T* o = out + (int64_t)dst * channels + head * HD + 4 * hf;
            u32x2 lo = {Half<T>::pack2(acc[0] * inv, acc[1] * inv), Half<T>::pack2(acc[2] * inv, acc[3] * inv)};
            u32x2 hi = {Half<T>::pack2(acc[4] * inv, acc[5] * inv), Half<T>::pack2(acc[6] * inv, acc[7] * inv)};
            *(u32x2*)o = lo;
            *(u32x2*)(o + 8) = hi;
            if (LSE && hf == 0) lse[(int64_t)head * lse_stride + s0 + qi] = acc[9] + __builtin_amdgcn_logf(acc[8]);
        }
    }
}

// ---- the general shape: thread per query, fp32 FMA arithmetic, chunks of K and V in LDS (as floats), any
// sequence length and head dims 8 ... 64. It serves fp32 (parity, the RPE path's sibling), and in half precision
// every shape the MFMA kernel above does not take: head dims other than 16 and sequences whose K and V do not
// fit its LDS. An order of magnitude slower than that kernel; there so that such models run at all.
constexpr int F32_QB = 256;        // queries per block
constexpr int F32_KV = 2048;       // floats of K (and of V) per chunk: 128 keys at head dim 16

template <typename T> __device__ __forceinline__ float any_to_float(T v) { return (float)v; }

template <typename T, int D>
__global__ __launch_bounds__(F32_QB) void patch_attn_any_kernel(
    const T* __restrict__ qkv, int channels, int heads, const int32_t* __restrict__ slot_src,
    const int32_t* __restrict__ slot_dst, const int32_t* __restrict__ cu_seqlens, int q_blocks,
    float scale, T* __restrict__ out, Dropout drop) {
    constexpr int KC = F32_KV / D;   // keys per chunk
    __shared__ float k_lds[KC][D];
    __shared__ float v_lds[KC][D];
    const int seq = blockIdx.x / (heads * q_blocks);
    const int rem = blockIdx.x % (heads * q_blocks);
    const int head = rem / q_blocks, qb = rem % q_blocks;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (qb * F32_QB >= len) return;
    const int tid = threadIdx.x;
    const int qi = qb * F32_QB + tid;
    const int64_t row_stride = 3 * (int64_t)channels;

    float q[D], o[D];
    int dst = -1;
#pragma unroll
    for (int d = 0; d < D; ++d) { q[d] = 0.f; o[d] = 0.f; }
    if (qi < len) {
        dst = slot_dst[s0 + qi];
        const T* src = qkv + (int64_t)slot_src[s0 + qi] * row_stride + head * D;
#pragma unroll
        for (int d = 0; d < D; ++d) q[d] = any_to_float(src[d]) * scale;
    }
    const uint32_t hq = drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + qi));
    float m = -INFINITY, l = 0.f;
    for (int c0 = 0; c0 < len; c0 += KC) {
        __syncthreads();
        for (int e = tid; e < KC * D; e += F32_QB) {
            const int key = e / D, d = e % D;
            float kv = 0.f, vv = 0.f;
            if (c0 + key < len) {
                const T* src = qkv + (int64_t)slot_src[s0 + c0 + key] * row_stride + head * D + d;
                kv = any_to_float(src[channels]);
                vv = any_to_float(src[2 * channels]);
            }
            k_lds[key][d] = kv;
            v_lds[key][d] = vv;
        }
        __syncthreads();
        const int kn = min(KC, len - c0);
        for (int key = 0; key < kn; ++key) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) s = fmaf(q[d], k_lds[key][d], s);
            if (s > m) {
                const float a = __expf(m - s);
                l *= a;
#pragma unroll
                for (int d = 0; d < D; ++d) o[d] *= a;
                m = s;
            }
            float p = __expf(s - m);
            l += p;
            if (drop.threshold && !drop_keep(hq, (uint32_t)(s0 + c0 + key), drop.threshold)) p = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) o[d] = fmaf(p, v_lds[key][d], o[d]);
        }
    }
    if (dst >= 0) {
        const float inv = drop.inv_keep / l;
        T* dstp = out + (int64_t)dst * channels + head * D;
#pragma unroll
        for (int d = 0; d < D; ++d) dstp[d] = (T)(o[d] * inv);
    }
}

// the head dims the thread-per-query kernels are instantiated for
bool any_head_dim(int d) { return d == 8 || d == 16 || d == 32 || d == 64; }

// the general kernel for (dtype, head dim); PTV3_ESHAPE for a head dim outside 8, 16, 32, 64
template <typename T>
int launch_any_t(const void* qkv, int channels, int heads, const int32_t* slot_src, const int32_t* slot_dst,
                 const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen, float scale, void* out, Dropout drop,
                 hipStream_t stream) {
    const int q_blocks = (int)ptv3_ceil_div(max_seqlen, F32_QB);
    if (n_seq * heads * q_blocks >= (1ll << 31)) return PTV3_EINVAL;
    const dim3 grid((unsigned)(n_seq * heads * q_blocks));
#define PTV3_ANY(D)                                                                                              \
    case D:                                                                                                      \
        hipLaunchKernelGGL((patch_attn_any_kernel<T, D>), grid, dim3(F32_QB), 0, stream, (const T*)qkv, channels, \
                           heads, slot_src, slot_dst, cu_seqlens, q_blocks, scale, (T*)out, drop);                \
        break;
    switch (channels / heads) {
        PTV3_ANY(8) PTV3_ANY(16) PTV3_ANY(32) PTV3_ANY(64)
        default: return PTV3_ESHAPE;
    }
#undef PTV3_ANY
    PTV3_RETURN_LAUNCH();
}

int launch_any(const void* qkv, int dtype, int channels, int heads, const int32_t* slot_src, const int32_t* slot_dst,
               const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen, float scale, void* out, Dropout drop,
               hipStream_t stream) {
    if (dtype == PTV3_F16)
        return launch_any_t<_Float16>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out,
                                      drop, stream);
    if (dtype == PTV3_BF16)
        return launch_any_t<__bf16>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out,
                                    drop, stream);
    return launch_any_t<float>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out, drop,
                               stream);
}

// ---- fp32 with relative position bias (model.py:297-316, :468-469): as above, and every score
// gets table[clamp(dx) + b][h] + table[R + clamp(dy) + b][h] + table[2R + clamp(dz) + b][h] for the
// grid offset (dx, dy, dz) = query - key, b = pos_bnd, R = 2 b + 1. The head's 3R table entries and
// the chunk's key coordinates sit in LDS.
constexpr int RPE_MAX_BND = 128;

template <int D>
__global__ __launch_bounds__(F32_QB) void patch_attn_rpe_f32_kernel(
    const float* __restrict__ qkv, int channels, int heads, const int32_t* __restrict__ slot_src,
    const int32_t* __restrict__ slot_dst, const int32_t* __restrict__ cu_seqlens, int q_blocks,
    float scale, const int32_t* __restrict__ grid_coord, const float* __restrict__ rpe_table, int pos_bnd,
    float* __restrict__ out, Dropout drop) {
    constexpr int KC = F32_KV / D;   // keys per chunk
    __shared__ float k_lds[KC][D];
    __shared__ float v_lds[KC][D];
    __shared__ int32_t c_lds[KC][3];
    __shared__ float t_lds[3 * (2 * RPE_MAX_BND + 1)];
    const int seq = blockIdx.x / (heads * q_blocks);
    const int rem = blockIdx.x % (heads * q_blocks);
    const int head = rem / q_blocks, qb = rem % q_blocks;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (qb * F32_QB >= len) return;
    const int tid = threadIdx.x;
    const int qi = qb * F32_QB + tid;
    const int64_t row_stride = 3 * (int64_t)channels;
    const int rnum = 2 * pos_bnd + 1;
    for (int e = tid; e < 3 * rnum; e += F32_QB) t_lds[e] = rpe_table[(int64_t)e * heads + head];

    float q[D], o[D];
    int dst = -1, qx = 0, qy = 0, qz = 0;
#pragma unroll
    for (int d = 0; d < D; ++d) { q[d] = 0.f; o[d] = 0.f; }
    if (qi < len) {
        dst = slot_dst[s0 + qi];
        const int64_t r = slot_src[s0 + qi];
        const float* src = qkv + r * row_stride + head * D;
#pragma unroll
        for (int d = 0; d < D; ++d) q[d] = src[d] * scale;
        qx = grid_coord[3 * r];
        qy = grid_coord[3 * r + 1];
        qz = grid_coord[3 * r + 2];
    }
    const uint32_t hq = drop_hq(drop.seed, (uint32_t)head, (uint32_t)(s0 + qi));
    float m = -INFINITY, l = 0.f;
    for (int c0 = 0; c0 < len; c0 += KC) {
        __syncthreads();
        for (int e = tid; e < KC * D; e += F32_QB) {
            const int key = e / D, d = e % D;
            float kv = 0.f, vv = 0.f;
            if (c0 + key < len) {
                const int64_t r = slot_src[s0 + c0 + key];
                const float* src = qkv + r * row_stride + head * D + d;
                kv = src[channels];
                vv = src[2 * channels];
                if (d < 3) c_lds[key][d] = grid_coord[3 * r + d];
            }
            k_lds[key][d] = kv;
            v_lds[key][d] = vv;
        }
        __syncthreads();
        const int kn = min(KC, len - c0);
        for (int key = 0; key < kn; ++key) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) s = fmaf(q[d], k_lds[key][d], s);
            const int dx = min(max(qx - c_lds[key][0], -pos_bnd), pos_bnd) + pos_bnd;
            const int dy = min(max(qy - c_lds[key][1], -pos_bnd), pos_bnd) + pos_bnd;
            const int dz = min(max(qz - c_lds[key][2], -pos_bnd), pos_bnd) + pos_bnd;
            s += t_lds[dx] + t_lds[rnum + dy] + t_lds[2 * rnum + dz];
            if (s > m) {
                const float a = __expf(m - s);
                l *= a;
#pragma unroll
                for (int d = 0; d < D; ++d) o[d] *= a;
                m = s;
            }
            float p = __expf(s - m);
            l += p;
            if (drop.threshold && !drop_keep(hq, (uint32_t)(s0 + c0 + key), drop.threshold)) p = 0.f;
#pragma unroll
            for (int d = 0; d < D; ++d) o[d] = fmaf(p, v_lds[key][d], o[d]);
        }
    }
    if (dst >= 0) {
        const float inv = drop.inv_keep / l;
        float* dstp = out + (int64_t)dst * channels + head * D;
#pragma unroll
        for (int d = 0; d < D; ++d) dstp[d] = o[d] * inv;
    }
}

// LDS of the MFMA kernel for sequences of up to max_seqlen keys: K (+ one prefetch-only step), V^T, per-step key
// norms (padded to 16 B), ones and zeros. Beyond 160 KB (2368 keys) the sequence does not fit.
size_t half_lds_bytes(int64_t max_seqlen) {
    const int64_t lds_keys = (max_seqlen + 63) & ~63ll;
    return (size_t)(lds_keys + 64) * 32 + (size_t)HD * (lds_keys * 2 + VT_PAD_BYTES) + (size_t)(lds_keys / 64) * sizeof(float) +
           12 + 192;
}
bool half_kernel_takes(int dtype, int channels, int heads, int64_t max_seqlen) {
    return dtype != PTV3_F32 && channels / heads == HD && half_lds_bytes(max_seqlen) <= 160 * 1024;
}

template <typename T, bool LSE, bool DROP>
int launch_half(const void* qkv, int channels, int heads, const int32_t* slot_src,
                const int32_t* slot_dst, const int32_t* cu_seqlens, int64_t n_seq,
                int64_t max_seqlen, float scale, void* out, float* lse, int64_t lse_stride, Dropout drop,
                hipStream_t stream) {
    const int lds_keys = (int)((max_seqlen + 63) & ~63ll);
    const size_t lds = half_lds_bytes(max_seqlen);
    if (lds > 160 * 1024) return PTV3_ESHAPE;
    auto kern = patch_attn_half_kernel<T, LSE, DROP>;
    static LdsGrant grant_lds_allowed;   // per instantiation and device; raised monotonically
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_lds_allowed)) return rc_;
    const float scale_log2e = scale * 1.4426950408889634f;
    // resident work-groups: two per CU (LDS-bound)
    static int slots = 0;
    if (slots == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        slots = 2 * cus;
    }
    // Items beyond the last full round of resident work-groups are cut into `split` query ranges
    // (each re-stages K/V, about a tenth of an item): pick the split that makes the tail shortest.
    const int64_t total = n_seq * heads;
    const int64_t rem = total % slots;
    int64_t full = total - rem, split = 1;
    if (rem != 0) {
        double best = 1.0;
        for (int64_t sp = 2; sp <= 4; ++sp) {
            const double cost = (double)((rem * sp + slots - 1) / slots) / (double)sp + 0.1;
            if (cost < best - 1e-9) { best = cost; split = sp; }
        }
    }
    if (split == 1) full = total;
    const int64_t tail = (total - full + 7) / 8 * 8;   // the tail's items in groups of 8, one per XCD
    hipLaunchKernelGGL(kern, dim3((unsigned)(full + tail * split)), dim3(ATT_THREADS), lds, stream,
                       (const T*)qkv, channels, heads, slot_src, slot_dst, cu_seqlens, lds_keys,
                       scale_log2e, (T*)out, (int)full, (int)split, (int)total, lse, lse_stride, drop);
    PTV3_RETURN_LAUNCH();
}

}  // namespace

extern "C" int ptv3_patch_attn_fwd(const void* qkv, int dtype, int64_t n_rows, int channels,
                                   int heads, const int32_t* slot_src, const int32_t* slot_dst,
                                   const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen,
                                   float scale, void* out, void* stream_) {
    if (n_rows < 0 || n_seq < 0 || channels < 1 || heads < 1 || max_seqlen < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (channels % heads != 0 || !any_head_dim(channels / heads)) return PTV3_ESHAPE;
    if (n_seq * heads >= (1ll << 31)) return PTV3_EINVAL;
    if (n_seq == 0 || n_rows == 0) return PTV3_OK;
    if (!qkv || !slot_src || !slot_dst || !cu_seqlens || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (half_kernel_takes(dtype, channels, heads, max_seqlen)) {
        if (dtype == PTV3_F16)
            return launch_half<_Float16, false, false>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                                       max_seqlen, scale, out, nullptr, 0, Dropout{0u, 0u, 1.f}, stream);
        return launch_half<__bf16, false, false>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                                 max_seqlen, scale, out, nullptr, 0, Dropout{0u, 0u, 1.f}, stream);
    }
    // fp32, and in half precision other head dims (8, 32, 64) or sequences beyond the MFMA kernel's LDS
    return launch_any(qkv, dtype, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out,
                      Dropout{0u, 0u, 1.f}, stream);
}

extern "C" int ptv3_patch_attn_fwd_lse(const void* qkv, int dtype, int64_t n_rows, int channels, int heads,
                                       const int32_t* slot_src, const int32_t* slot_dst, const int32_t* cu_seqlens,
                                       int64_t n_seq, int64_t max_seqlen, int64_t n_pad, float scale, float dropout_p,
                                       uint32_t dropout_seed, void* out, float* lse, void* stream_) {
    if (n_rows < 0 || n_seq < 0 || n_pad < 0 || channels < 1 || heads < 1 || max_seqlen < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16 || !(dropout_p >= 0.f) || !(dropout_p < 1.f)) return PTV3_EINVAL;
    if (channels % heads != 0 || channels / heads != HD) return PTV3_ESHAPE;
    if (n_seq * heads >= (1ll << 31)) return PTV3_EINVAL;
    if (n_seq == 0 || n_rows == 0) return PTV3_OK;
    if (!qkv || !slot_src || !slot_dst || !cu_seqlens || !out || (dtype != PTV3_F32 && !lse)) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    const Dropout drop = {dropout_seed, dropout_p > 0.f ? drop_threshold(dropout_p) : 0u, 1.f / (1.f - dropout_p)};
    if (dtype == PTV3_F32)   // the backward recomputes the log-sum-exp rows on this path
        return launch_any(qkv, dtype, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out, drop,
                          stream);
#define PTV3_ATT(T, D)                                                                                               \
    return launch_half<T, true, D>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq, max_seqlen, scale, out, \
                                   lse, n_pad, drop, stream)
    if (dtype == PTV3_F16) {
        if (drop.threshold) PTV3_ATT(_Float16, true);
        PTV3_ATT(_Float16, false);
    }
    if (drop.threshold) PTV3_ATT(__bf16, true);
    PTV3_ATT(__bf16, false);
#undef PTV3_ATT
}

extern "C" int ptv3_patch_attn_rpe_fwd(const float* qkv, int64_t n_rows, int channels, int heads,
                                       const int32_t* slot_src, const int32_t* slot_dst,
                                       const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen, float scale,
                                       const int32_t* grid_coord, const float* rpe_table, int pos_bnd, float dropout_p,
                                       uint32_t dropout_seed, float* out, void* stream_) {
    if (!(dropout_p >= 0.f) || !(dropout_p < 1.f)) return PTV3_EINVAL;
    const Dropout drop = {dropout_seed, dropout_p > 0.f ? drop_threshold(dropout_p) : 0u, 1.f / (1.f - dropout_p)};
    if (n_rows < 0 || n_seq < 0 || channels < 1 || heads < 1 || max_seqlen < 1) return PTV3_EINVAL;
    if (pos_bnd < 0 || pos_bnd > RPE_MAX_BND) return PTV3_ESHAPE;
    if (channels % heads != 0 || !any_head_dim(channels / heads)) return PTV3_ESHAPE;
    if (n_seq == 0 || n_rows == 0) return PTV3_OK;
    if (!qkv || !slot_src || !slot_dst || !cu_seqlens || !grid_coord || !rpe_table || !out) return PTV3_EINVAL;
    const int q_blocks = (int)ptv3_ceil_div(max_seqlen, F32_QB);
    if (n_seq * heads * q_blocks >= (1ll << 31)) return PTV3_EINVAL;
    const dim3 grid((unsigned)(n_seq * heads * q_blocks));
#define PTV3_RPE(D)                                                                                                  \
    case D:                                                                                                          \
        hipLaunchKernelGGL(patch_attn_rpe_f32_kernel<D>, grid, dim3(F32_QB), 0, (hipStream_t)stream_, qkv, channels, \
                           heads, slot_src, slot_dst, cu_seqlens, q_blocks, scale, grid_coord, rpe_table, pos_bnd, out, \
                           drop);                                                                                    \
        break;
    switch (channels / heads) {
        PTV3_RPE(8) PTV3_RPE(16) PTV3_RPE(32) PTV3_RPE(64)
        default: return PTV3_ESHAPE;
    }
#undef PTV3_RPE
    PTV3_RETURN_LAUNCH();
}
