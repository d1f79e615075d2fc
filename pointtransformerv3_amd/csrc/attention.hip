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
//   * V^T only fills 16 of the 32 rows of that product; rows 16 and 20 are fed ones so the
//     softmax denominator falls out of the same MFMA instead of costing VALU adds.
//   * Rows are read through slot_src and written through slot_dst, so the padded,
//     permuted qkv tensor of the reference is never materialised.
// fp32 kernel: one thread per query, K/V chunks staged in LDS, plain FMA arithmetic.
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

constexpr int HD = 16;             // head dim
constexpr int ATT_THREADS = 256;   // 4 waves
constexpr int ATT_WAVES = ATT_THREADS / PTV3_WAVE;
constexpr int VT_PAD_BYTES = 16;   // skews V^T rows across LDS banks

template <typename T> struct Half;
template <> struct Half<_Float16> {
    typedef f16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        f16x2 h = __builtin_convertvector(f, f16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ uint16_t one() { return 0x3C00; }
};
template <> struct Half<__bf16> {
    typedef bf16x8 v8;
    static __device__ __forceinline__ f32x16 mfma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        f32x2 f = {a, b};
        bf16x2 h = __builtin_convertvector(f, bf16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ uint16_t one() { return 0x3F80; }
};

// position of key kk (0..31) inside its 32-key block of the transposed V tile: the keys a
// lane of half h holds in result registers 0..15 are 8*(v/4) + 4*h + v%4.
__device__ __forceinline__ int vt_pos(int kk) {
    return ((kk >> 2) & 1) * 16 + (kk >> 3) * 4 + (kk & 3);
}

template <typename T>
__global__ __launch_bounds__(ATT_THREADS, 2) void patch_attn_half_kernel(
    const T* __restrict__ qkv, int channels, int heads, const int32_t* __restrict__ slot_src,
    const int32_t* __restrict__ slot_dst, const int32_t* __restrict__ cu_seqlens, int lds_keys,
    float scale_log2e, T* __restrict__ out) {
    typedef typename Half<T>::v8 v8;
    extern __shared__ __align__(16) unsigned char smem[];
    // K tile: lds_keys rows of 32 B. V^T tile: 16 rows of (lds_keys*2 + pad) B.
    unsigned char* k_lds = smem;
    const int vt_stride = lds_keys * 2 + VT_PAD_BYTES;
    unsigned char* vt_lds = smem + (size_t)lds_keys * 32;

    const int seq = blockIdx.x / heads, head = blockIdx.x % heads;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (len <= 0) return;
    const int len32 = (len + 31) & ~31;
    const int tid = threadIdx.x;
    const int64_t row_stride = 3 * (int64_t)channels;

    // ---- stage K and V^T: thread handles (key, 8-channel half)
    for (int e = tid; e < len32 * 2; e += ATT_THREADS) {
        const int key = e >> 1, part = e & 1;
        u32x4 kq = {0, 0, 0, 0}, vq = {0, 0, 0, 0};
        if (key < len) {
            const T* base = qkv + (int64_t)slot_src[s0 + key] * row_stride + head * HD + part * 8;
            kq = *(const u32x4*)(base + channels);
            vq = *(const u32x4*)(base + 2 * channels);
        }
        *(u32x4*)(k_lds + key * 32 + part * 16) = kq;
        const int pos = (key & ~31) + vt_pos(key & 31);
        uint16_t* vt = (uint16_t*)(vt_lds + (size_t)(part * 8) * vt_stride) + pos;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w = vq[c];
            *(uint16_t*)((unsigned char*)vt + (size_t)(2 * c) * vt_stride) = (uint16_t)(w & 0xffffu);
            *(uint16_t*)((unsigned char*)vt + (size_t)(2 * c + 1) * vt_stride) = (uint16_t)(w >> 16);
        }
    }
    __syncthreads();

    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int n_tiles = len32 / 32;

    // A operand rows of the second product: d < 16 read V^T, rows 16 and 20 are ones.
    u32x4 ones4;
    {
        const uint32_t o = (col == 16 || col == 20) ? (Half<T>::one() * 0x10001u) : 0u;
        ones4 = (u32x4){o, o, o, o};
    }

    for (int qt = wave; qt < n_tiles; qt += ATT_WAVES) {
        const int qi = qt * 32 + col;   // my query inside the sequence
        int dst = -1;
        u32x4 qreg = {0, 0, 0, 0};
        if (qi < len) {
            dst = slot_dst[s0 + qi];
            qreg = *(const u32x4*)(qkv + (int64_t)slot_src[s0 + qi] * row_stride + head * HD + hf * 8);
        }
        if (__ballot(dst >= 0) == 0) continue;   // tile of filler slots only
        const v8 qfrag = __builtin_bit_cast(v8, qreg);

        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        float m = -INFINITY;   // running max of raw scores (same in lane and lane^32)

        for (int kt = 0; kt < n_tiles; ++kt) {
            const v8 kfrag = __builtin_bit_cast(v8, *(const u32x4*)(k_lds + (kt * 32 + col) * 32 + hf * 16));
            f32x16 s;
#pragma unroll
            for (int v = 0; v < 16; ++v) s[v] = 0.f;
            s = Half<T>::mfma(kfrag, qfrag, s);   // s[v] = <K[key_v], Q[q]>
            if (kt == n_tiles - 1 && len != len32) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = kt * 32 + 8 * (v >> 2) + 4 * hf + (v & 3);
                    if (key >= len) s[v] = -INFINITY;
                }
            }
            float mt = s[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) mt = fmaxf(mt, s[v]);
            mt = fmaxf(mt, __shfl_xor(mt, 32, PTV3_WAVE));
            const float m_new = fmaxf(m, mt);
            const float alpha = exp2f((m - m_new) * scale_log2e);
            const float mc = m_new * scale_log2e;
            m = m_new;
#pragma unroll
            for (int v = 0; v < 9; ++v) acc[v] *= alpha;   // rows 0..15 (+ the denominator row)
            uint32_t p[8];
#pragma unroll
            for (int v = 0; v < 8; ++v)
                p[v] = Half<T>::pack2(exp2f(fmaf(s[2 * v], scale_log2e, -mc)),
                                      exp2f(fmaf(s[2 * v + 1], scale_log2e, -mc)));
            u32x4 va = ones4, vb = ones4;
            if (col < HD) {
                const unsigned char* vrow = vt_lds + (size_t)col * vt_stride + (kt * 32 + hf * 16) * 2;
                va = *(const u32x4*)vrow;
                vb = *(const u32x4*)(vrow + 16);
            }
            const u32x4 pa = {p[0], p[1], p[2], p[3]}, pb = {p[4], p[5], p[6], p[7]};
            acc = Half<T>::mfma(__builtin_bit_cast(v8, va), __builtin_bit_cast(v8, pa), acc);
            acc = Half<T>::mfma(__builtin_bit_cast(v8, vb), __builtin_bit_cast(v8, pb), acc);
        }
        // acc[v]: d = 8*(v/4) + 4*hf + v%4; acc[8] = sum of probabilities (row 16 / 20)
        if (dst >= 0) {
            const float inv = 1.f / acc[8];
            T* o = out + (int64_t)dst * channels + head * HD + 4 * hf;
            u32x2 lo = {Half<T>::pack2(acc[0] * inv, acc[1] * inv), Half<T>::pack2(acc[2] * inv, acc[3] * inv)};
            u32x2 hi = {Half<T>::pack2(acc[4] * inv, acc[5] * inv), Half<T>::pack2(acc[6] * inv, acc[7] * inv)};
            *(u32x2*)o = lo;
            *(u32x2*)(o + 8) = hi;
        }
    }
}

// ---- fp32: thread per query, 128-key chunks of K and V in LDS.
constexpr int F32_QB = 256;   // queries per block
constexpr int F32_KC = 128;   // keys per chunk

__global__ __launch_bounds__(F32_QB) void patch_attn_f32_kernel(
    const float* __restrict__ qkv, int channels, int heads, const int32_t* __restrict__ slot_src,
    const int32_t* __restrict__ slot_dst, const int32_t* __restrict__ cu_seqlens, int q_blocks,
    float scale, float* __restrict__ out) {
    __shared__ float k_lds[F32_KC][HD];
    __shared__ float v_lds[F32_KC][HD];
    const int seq = blockIdx.x / (heads * q_blocks);
    const int rem = blockIdx.x % (heads * q_blocks);
    const int head = rem / q_blocks, qb = rem % q_blocks;
    const int s0 = cu_seqlens[seq];
    const int len = cu_seqlens[seq + 1] - s0;
    if (qb * F32_QB >= len) return;
    const int tid = threadIdx.x;
    const int qi = qb * F32_QB + tid;
    const int64_t row_stride = 3 * (int64_t)channels;

    float q[HD], o[HD];
    int dst = -1;
#pragma unroll
    for (int d = 0; d < HD; ++d) { q[d] = 0.f; o[d] = 0.f; }
    if (qi < len) {
        dst = slot_dst[s0 + qi];
        const float* src = qkv + (int64_t)slot_src[s0 + qi] * row_stride + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) q[d] = src[d] * scale;
    }
    float m = -INFINITY, l = 0.f;
    for (int c0 = 0; c0 < len; c0 += F32_KC) {
        __syncthreads();
        for (int e = tid; e < F32_KC * HD; e += F32_QB) {
            const int key = e / HD, d = e % HD;
            float kv = 0.f, vv = 0.f;
            if (c0 + key < len) {
                const float* src = qkv + (int64_t)slot_src[s0 + c0 + key] * row_stride + head * HD + d;
                kv = src[channels];
                vv = src[2 * channels];
            }
            k_lds[key][d] = kv;
            v_lds[key][d] = vv;
        }
        __syncthreads();
        const int kn = min(F32_KC, len - c0);
        for (int key = 0; key < kn; ++key) {
            float s = 0.f;
#pragma unroll
            for (int d = 0; d < HD; ++d) s = fmaf(q[d], k_lds[key][d], s);
            if (s > m) {
                const float a = __expf(m - s);
                l *= a;
#pragma unroll
                for (int d = 0; d < HD; ++d) o[d] *= a;
                m = s;
            }
            const float p = __expf(s - m);
            l += p;
#pragma unroll
            for (int d = 0; d < HD; ++d) o[d] = fmaf(p, v_lds[key][d], o[d]);
        }
    }
    if (dst >= 0) {
        const float inv = 1.f / l;
        float* dstp = out + (int64_t)dst * channels + head * HD;
#pragma unroll
        for (int d = 0; d < HD; ++d) dstp[d] = o[d] * inv;
    }
}

template <typename T>
int launch_half(const void* qkv, int channels, int heads, const int32_t* slot_src,
                const int32_t* slot_dst, const int32_t* cu_seqlens, int64_t n_seq,
                int64_t max_seqlen, float scale, void* out, hipStream_t stream) {
    const int lds_keys = (int)((max_seqlen + 31) & ~31ll);
    const size_t lds = (size_t)lds_keys * 32 + (size_t)HD * (lds_keys * 2 + VT_PAD_BYTES);
    if (lds > 160 * 1024) return PTV3_ESHAPE;
    auto kern = patch_attn_half_kernel<T>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    const float scale_log2e = scale * 1.4426950408889634f;
    hipLaunchKernelGGL(kern, dim3((unsigned)(n_seq * heads)), dim3(ATT_THREADS), lds, stream,
                       (const T*)qkv, channels, heads, slot_src, slot_dst, cu_seqlens, lds_keys,
                       scale_log2e, (T*)out);
    PTV3_RETURN_LAUNCH();
}

}  // namespace

extern "C" int ptv3_patch_attn_fwd(const void* qkv, int dtype, int64_t n_rows, int channels,
                                   int heads, const int32_t* slot_src, const int32_t* slot_dst,
                                   const int32_t* cu_seqlens, int64_t n_seq, int64_t max_seqlen,
                                   float scale, void* out, void* stream_) {
    if (n_rows < 0 || n_seq < 0 || channels < 1 || heads < 1 || max_seqlen < 1) return PTV3_EINVAL;
    if (dtype < PTV3_F32 || dtype > PTV3_BF16) return PTV3_EINVAL;
    if (channels % heads != 0 || channels / heads != HD) return PTV3_ESHAPE;
    if (n_seq * heads >= (1ll << 31)) return PTV3_EINVAL;
    if (n_seq == 0 || n_rows == 0) return PTV3_OK;
    if (!qkv || !slot_src || !slot_dst || !cu_seqlens || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16)
        return launch_half<_Float16>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                     max_seqlen, scale, out, stream);
    if (dtype == PTV3_BF16)
        return launch_half<__bf16>(qkv, channels, heads, slot_src, slot_dst, cu_seqlens, n_seq,
                                   max_seqlen, scale, out, stream);
    const int q_blocks = (int)ptv3_ceil_div(max_seqlen, F32_QB);
    if (n_seq * heads * q_blocks >= (1ll << 31)) return PTV3_EINVAL;
    hipLaunchKernelGGL(patch_attn_f32_kernel, dim3((unsigned)(n_seq * heads * q_blocks)), dim3(F32_QB),
                       0, stream, (const float*)qkv, channels, heads, slot_src, slot_dst, cu_seqlens,
                       q_blocks, scale, (float*)out);
    PTV3_RETURN_LAUNCH();
}
