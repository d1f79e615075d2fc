// Fused MLP for wide channels (C = 128, 256, 512; hidden = 4C; half precision):
//   out = resid + fc2(GELU(fc1(x)))                       (model.py:493-516, :599-602)
// As separate kernels this is three passes over an N x 4C tensor (fc1 writes it, GELU rewrites it,
// fc2 reads it); here a work-group keeps a tile of rows on the CU for the whole chain.
//
// The biases of both layers sit in LDS for the life of the work-group: a vector-memory load of them at the head of a
// chunk would have to wait for the weight fragments requested before it (loads return in order), draining the ring.
// A work-group of 8 waves owns R = 64 ... 192 rows (RT = 2 or 3 groups of 32 rows per wave). The hidden axis is cut into four chunks of C
// units; per chunk, stage A computes GELU(x W1_chunk^T + b1) for the tile into LDS and stage B adds
// its product with W2's chunk to the output accumulators, which stay in registers across the
// chunks. Products are taken transposed with v_mfma_f32_32x32x16 (rows of the A operand = output
// units, columns = points); a wave owns 64 points x 32*MT output units in both stages, reads the
// point-side operand from LDS (the x tile in stage A, the hidden chunk in stage B) and streams
// its own rows of W1 / W2 straight from L2 into operand registers, 64 contiguous bytes per weight
// row and step. No two waves of a work-group with the same points share weight rows, so nothing
// is fetched into LDS twice, and the weight stream runs DEPTH steps ahead in a ring of registers
// that is never drained: its addresses do not depend on the tile, so it runs on across stages,
// chunks and tiles of the persistent work-group.
// Read from the Linear layers' own (out, in) layout such a step touches 32 weight rows with 2 x 16 bytes each
// per instruction, and the texture path spends a cycle per lane and line on that: three to four times what a
// contiguous KB costs. ptv3_mlp_pack_weights therefore writes both matrices once in the order of the stream
// (step, 32-unit block, piece, lane), and the PACKED kernel fetches every fragment as one contiguous KB.
// Intermediates are rounded to the storage type where the separate layers would have stored them.
// The same kernel has two more modes at 128 and 256 channels (TAIL_MODE, HEAD_MODE below): the halves of a block in
// front of and behind its attention, with the projection / the xCPE's Linear and their LayerNorms as further stages
// of a pass (model.py:541-545, :587-602).
#include <type_traits>

#include "rowtile.h"

namespace {

constexpr int MW_THREADS = 512;
constexpr int MW_PAD = 8;   // halfs of padding per LDS row

// weight step u of the stream (UNITS = 8 C / 32 of them): chunk u / (2 KU), stage (u / KU) & 1 (fc1, fc2), 32-wide
// contraction step kk = u % KU with KU = C / 32. Piece j of lane (col, hf) for the 32-unit block ub holds inputs
// 32 kk + 16 hf + 8 j .. + 8 of unit 32 ub + col: row chunk C + unit of fc1, or row unit of fc2 from column chunk C on.
// packed[((u * (C / 32) + ub) * 2 + j) * 512 + lane * 8 .. + 8]
template <typename T>
__global__ __launch_bounds__(256) void mlp_pack_kernel(const T* __restrict__ w1, const T* __restrict__ w2, int c,
                                                        T* __restrict__ packed) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;   // one 16-byte piece each
    if (idx >= (int64_t)c * c) return;                            // 8 C^2 elements in pieces of 8
    const int lane = (int)(idx % 64), j = (int)(idx / 64 % 2), ub = (int)(idx / 128 % (c / 32));
    const int u = (int)(idx / 128 / (c / 32)), ku = c / 32;
    const int chunk = u / (2 * ku), st = (u / ku) & 1, kk = u % ku;
    const int unit = ub * 32 + lane % 32, k = kk * 32 + (lane / 32) * 16 + j * 8;
    const T* src = st == 0 ? w1 + (int64_t)(chunk * c + unit) * c + k : w2 + (int64_t)unit * 4 * c + chunk * c + k;
    *(u32x4*)(packed + idx * 8) = *(const u32x4*)src;
}

// the same for several MLPs in one launch: job j owns blocks first_block[j] .. first_block[j + 1]
__global__ __launch_bounds__(256) void mlp_pack_batch_kernel(const ptv3_mlp_pack_job* __restrict__ jobs, int n_jobs) {
    int j = 0;
    for (int i = 1; i < n_jobs; ++i)
        if (jobs[i].first_block <= (int64_t)blockIdx.x) j = i;   // uniform: a handful of jobs, first_block ascending
    const ptv3_mlp_pack_job job = jobs[j];
    const int c = job.channels;
    if (c != 128 && c != 256 && c != 512) return;   // a width the fused kernel does not take: touch nothing
    const int64_t idx = ((int64_t)blockIdx.x - job.first_block) * 256 + threadIdx.x;
    // a job without w2 is a (k C, C) matrix of k = max(reserved, 1) chunks of C rows, every chunk like a chunk of fc1
    const int k_chunks = job.reserved > 0 ? job.reserved : 1;
    if (idx < 0 || idx >= (job.w2 ? (int64_t)c * c : (int64_t)k_chunks * c * c / 8)) return;
    const int lane = (int)(idx % 64), jj = (int)(idx / 64 % 2), ub = (int)(idx / 128 % (c / 32));
    const int u = (int)(idx / 128 / (c / 32)), ku = c / 32;
    const int chunk = job.w2 ? u / (2 * ku) : u / ku, st = job.w2 ? (u / ku) & 1 : 0, kk = u % ku;
    const int unit = ub * 32 + lane % 32, k = kk * 32 + (lane / 32) * 16 + jj * 8;
    const uint16_t *w1 = (const uint16_t*)job.w1, *w2 = (const uint16_t*)job.w2;   // both half types: 16-bit patterns
    const uint16_t* src = st == 0 ? w1 + (int64_t)(chunk * c + unit) * c + k : w2 + (int64_t)unit * 4 * c + chunk * c + k;
    *(u32x4*)((uint16_t*)job.packed + idx * 8) = *(const u32x4*)src;
}

// PACKED: w1 is the packed stream of both matrices and w2 is not read.
// TAIL (PACKED only): the whole second half of a block. x is the attention's output, resid the block's running sum; a
// pass first forms sum = resid + (x Wp^T + bp) and LayerNorm(sum) on the CU (wp: Wp packed like fc1's first chunk,
// the stream then has KU steps more at its head), feeds the normalised rows to the MLP and adds the MLP to the sum,
// which waits in a third LDS tile: neither the sum nor its normalised copy travels to memory and back.
// A work-group walks its rows in passes of 1 .. RTMAX groups of 32 rows per wave; the host gives every resident
// work-group the same number of row groups (with tiles of one fixed size the last round of a launch of 37,681 rows at
// 256 channels ran at half occupancy).
// HEAD_MODE (PACKED only): the first half of a block behind its convolution. x is the convolution's output, resid the
// block's input; a pass forms sum = resid + LayerNorm_cpe(x Wc^T + bc), writes it to out, and multiplies
// LayerNorm_1(sum) by the three C-row chunks of the qkv weight (w1: Wc and Wqkv packed one behind the other, 4 KU
// steps a pass), writing (N, 3C) rows to extra.qkv: the normalised rows never travel to memory and back.
struct WideArgs {   // what the block halves add to the MLP's arguments
    const void *wp, *bp, *ln_w, *ln_b;   // TAIL: packed projection, its bias; LayerNorm_2. HEAD: -, bc; LayerNorm_cpe
    float eps;
    const void *ln1_w, *ln1_b, *bq;      // HEAD: LayerNorm_1, the qkv bias (3C)
    float eps1;
    void* qkv;                           // HEAD: (N, 3C) out
};
constexpr int MLP_MODE = 0, TAIL_MODE = 1, HEAD_MODE = 2;

template <typename T, int C, int WM, int WN, int MT, int DEPTH, bool PACKED, int RTMAX, int THREADS, int MINW, int MODE>
__global__ __launch_bounds__(THREADS, MINW) void mlp_wide_kernel(
    const T* __restrict__ x, const T* __restrict__ resid, const T* __restrict__ w1, const T* __restrict__ b1,
    const T* __restrict__ w2, const T* __restrict__ b2, int64_t n, int upw, T* __restrict__ out, WideArgs extra) {
    constexpr bool TAIL = MODE == TAIL_MODE, HEADM = MODE == HEAD_MODE;
    static_assert(MODE == MLP_MODE || PACKED, "the block halves read packed weights");
    typedef typename H16<T>::v8 v8;
    static_assert(WM * WN * PTV3_WAVE == THREADS && C == 32 * MT * WN, "the waves cover R x C");
    constexpr int RMAX = 32 * RTMAX * WM, H = 4 * C, XS = C + MW_PAD;
    constexpr int KU = C / 32;            // 32-wide contraction steps per stage
    constexpr int FRONT = TAIL ? KU : 0;  // weight steps of the projection in front of the MLP's
    // weight steps per pass: (projection,) 4 chunks x (fc1, fc2); HEAD: the xCPE's Linear and three chunks of qkv
    constexpr int UNITS = HEADM ? 4 * KU : FRONT + 4 * 2 * KU;
    static_assert(KU % DEPTH == 0, "the ring is indexed statically");
    constexpr int PPR = C / 8;            // 16-byte pieces per row
    extern __shared__ __align__(16) unsigned char mw_smem[];
    T* xt = (T*)mw_smem;                  // [RMAX][XS] input tile
    T* ht = xt + RMAX * XS;               // [RMAX][XS] hidden chunk, then the output tile
    T* bias_lds = ht + RMAX * XS;         // [4 C] fc1's bias, [C] fc2's: read per chunk without touching the vector-memory queue
    if (!HEADM)
        for (int i = threadIdx.x; i < 5 * C / 8; i += THREADS)
            *(u32x4*)(bias_lds + i * 8) = *(const u32x4*)((i < 4 * C / 8 ? b1 : b2 - 4 * C) + i * 8);
    if (HEADM)   // [C] each: the xCPE Linear's bias, LayerNorm_cpe's scale and shift, LayerNorm_1's; [3 C] the qkv bias
        for (int i = threadIdx.x; i < 8 * C / 8; i += THREADS) {
            const int which = i / (C / 8), at = i % (C / 8);
            const T* src = (const T*)(which == 0 ? extra.bp : which == 1 ? extra.ln_w : which == 2 ? extra.ln_b
                                      : which == 3 ? extra.ln1_w : which == 4 ? extra.ln1_b : extra.bq);
            *(u32x4*)(bias_lds + i * 8) = *(const u32x4*)(src + (which >= 5 ? i - 5 * (C / 8) : at) * 8);
        }
    T* sum_lds = bias_lds + 8 * C;        // TAIL: [RMAX][XS] the block's running sum (HEAD: a second staging tile); before it the projection's bias
    if (TAIL)                             // and the LayerNorm's scale and shift, [C] each
        for (int i = threadIdx.x; i < 3 * C / 8; i += THREADS) {
            const int which = i / (C / 8), at = i % (C / 8);
            const T* src = (const T*)(which == 0 ? extra.bp : which == 1 ? extra.ln_w : extra.ln_b);
            *(u32x4*)(bias_lds + 5 * C + i * 8) = *(const u32x4*)(src + at * 8);
        }

    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int wm = wave % WM, wn = wave / WM;
    const int ch0 = wn * 32 * MT;   // first output unit of this wave (hidden unit inside a chunk / channel)

    // weight step q of a pass: chunk q / (2 KU), layer (q / KU) & 1 (fc1, fc2), 32-wide step kk = q % KU; lane (col, hf)
    // of output tile a takes 2 x 8 consecutive inputs of weight row ch0 + 32 a + col
    auto issue = [&](int q, u32x4 (&r)[MT][2]) {
        const int u = TAIL && q < FRONT ? q : q - FRONT;   // step inside its own packed copy
        const int chunk = u / (2 * KU), st = (u / KU) & 1, kk = u % KU;
#pragma unroll
        for (int a = 0; a < MT; ++a) {
            if (PACKED) {
                const T* p = (TAIL && q < FRONT ? (const T*)extra.wp : w1) + ((u * (C / 32) + wn * MT + a) * 2) * 512 + lane * 8;
                r[a][0] = *(const u32x4*)p;
                r[a][1] = *(const u32x4*)(p + 512);
                continue;
            }
            const int unit = ch0 + a * 32 + col;
            const T* p = st == 0 ? w1 + (int64_t)(chunk * C + unit) * C + kk * 32 + hf * 16
                                 : w2 + (int64_t)unit * H + chunk * C + kk * 32 + hf * 16;
            r[a][0] = *(const u32x4*)p;
            r[a][1] = *(const u32x4*)(p + 8);
        }
    };
    u32x4 ring[DEPTH][MT][2];
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) issue(j, ring[j]);

    // one pass over RT_ row groups per wave, rows [row0, row0 + 32 RT_ WM) of which those below row_end exist
    auto pass = [&](auto rt_c, int64_t row0, int64_t row_end) {
        constexpr int RT_ = decltype(rt_c)::value;
        constexpr int PIECES = 32 * RT_ * WM * PPR / THREADS;
        const int r0 = wm * 32 * RT_;    // first row of this wave inside the tile

        // one matrix stage: acc[a][rt] += W rows (ring) x tile rows (LDS `src`); q0 = its first weight step
        auto stage = [&](const T* src, f32x16 (&acc)[MT][RT_], int q0) {
            const T* brow = src + (r0 + col) * XS + hf * 16;
#pragma unroll
            for (int kk = 0; kk < KU; ++kk) {
                const int j = kk % DEPTH;
                u32x4 bf[RT_][2];
#pragma unroll
                for (int rt = 0; rt < RT_; ++rt) {
                    bf[rt][0] = *(const u32x4*)(brow + rt * 32 * XS + kk * 32);
                    bf[rt][1] = *(const u32x4*)(brow + rt * 32 * XS + kk * 32 + 8);
                }
                u32x4 af[MT][2];
#pragma unroll
                for (int a = 0; a < MT; ++a) {
                    af[a][0] = ring[j][a][0];
                    af[a][1] = ring[j][a][1];
                }
                int qn = q0 + kk + DEPTH;
                if (qn >= UNITS) qn -= UNITS;   // the stream of the next pass is the same
                issue(qn, ring[j]);
#pragma unroll
                for (int a = 0; a < MT; ++a)
#pragma unroll
                    for (int rt = 0; rt < RT_; ++rt) {
                        acc[a][rt] = H16<T>::mfma(__builtin_bit_cast(v8, af[a][0]), __builtin_bit_cast(v8, bf[rt][0]), acc[a][rt]);
                        acc[a][rt] = H16<T>::mfma(__builtin_bit_cast(v8, af[a][1]), __builtin_bit_cast(v8, bf[rt][1]), acc[a][rt]);
                    }
            }
        };
        // fc1's sums start from its bias (the MFMAs' C operand) instead of having it added afterwards
        auto bias_into = [&](f32x16 (&hacc)[MT][RT_], int chunk) {
#pragma unroll
            for (int a = 0; a < MT; ++a)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const u32x2 bb = *(const u32x2*)(bias_lds + chunk * C + ch0 + a * 32 + 8 * g + 4 * hf);
                    const float bias[4] = {H16<T>::lo(bb[0]), H16<T>::hi(bb[0]), H16<T>::lo(bb[1]), H16<T>::hi(bb[1])};
#pragma unroll
                    for (int rt = 0; rt < RT_; ++rt)
#pragma unroll
                        for (int q = 0; q < 4; ++q) hacc[a][rt][4 * g + q] = bias[q];
                }
        };
        // ---- x tile -> LDS
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int p = tid + i * THREADS;
            const int rr = p / PPR, pc = p % PPR;
            u32x4 v = {0, 0, 0, 0}, sh = {0, 0, 0, 0};
            if (row0 + rr < row_end) {
                v = *(const u32x4*)(x + (row0 + rr) * C + pc * 8);
                if (TAIL) sh = *(const u32x4*)(resid + (row0 + rr) * C + pc * 8);   // waits in LDS for the projection
            }
            *(u32x4*)(xt + rr * XS + pc * 8) = v;
            if (TAIL) *(u32x4*)(sum_lds + rr * XS + pc * 8) = sh;
        }
        __syncthreads();

        f32x16 acc[MT][RT_], hacc[MT][RT_];
        // sums start from a bias vector in LDS (the MFMAs' C operand)
        auto bias_from = [&](f32x16 (&sums)[MT][RT_], const T* vec) {
#pragma unroll
            for (int a = 0; a < MT; ++a)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const u32x2 bb = *(const u32x2*)(vec + ch0 + a * 32 + 8 * g + 4 * hf);
                    const float bias[4] = {H16<T>::lo(bb[0]), H16<T>::hi(bb[0]), H16<T>::lo(bb[1]), H16<T>::hi(bb[1])};
#pragma unroll
                    for (int rt = 0; rt < RT_; ++rt)
#pragma unroll
                        for (int q = 0; q < 4; ++q) sums[a][rt][4 * g + q] = bias[q];
                }
        };
        // the wave's sums, rounded, into the staging tile
        auto park = [&](const f32x16 (&sums)[MT][RT_], T* tile) {
#pragma unroll
            for (int a = 0; a < MT; ++a)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int cc = ch0 + a * 32 + 8 * g + 4 * hf;
#pragma unroll
                    for (int rt = 0; rt < RT_; ++rt)
                        *(u32x2*)(tile + (r0 + rt * 32 + col) * XS + cc) =
                            (u32x2){H16<T>::pack2(sums[a][rt][4 * g], sums[a][rt][4 * g + 1]),
                                    H16<T>::pack2(sums[a][rt][4 * g + 2], sums[a][rt][4 * g + 3])};
                }
        };
        // LayerNorm of a row whose PPR pieces of 8 values sit in neighbouring lanes of one wave (the statistics are
        // lane exchanges): v (this lane's piece) -> its normalised, scaled and shifted values, rounded and packed
        auto norm_piece = [&](float (&v)[8], const u32x4 gq, const u32x4 bq, float eps) -> u32x4 {
            float tot = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) tot += v[k];
#pragma unroll
            for (int off = 1; off < PPR; off <<= 1) tot += __shfl_xor(tot, off, PTV3_WAVE);
            const float mean = tot * (1.f / C);
            float sq = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                v[k] -= mean;
                sq += v[k] * v[k];
            }
#pragma unroll
            for (int off = 1; off < PPR; off <<= 1) sq += __shfl_xor(sq, off, PTV3_WAVE);
            const float rstd = rsqrtf(sq * (1.f / C) + eps);
            u32x4 nm;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                nm[k] = H16<T>::pack2(v[2 * k] * rstd * H16<T>::lo(gq[k]) + H16<T>::lo(bq[k]),
                                      v[2 * k + 1] * rstd * H16<T>::hi(gq[k]) + H16<T>::hi(bq[k]));
            return nm;
        };
        if constexpr (TAIL) {
            // ---- projection of the attention rows (+ bias), rounded, parked in ht
            bias_from(hacc, bias_lds + 5 * C);
            stage(xt, hacc, 0);
            park(hacc, ht);
            __syncthreads();   // every wave is done reading the attention rows in xt, the projection is in ht
            // ---- sum = resid + projection (rounded, kept in sum_lds); its LayerNorm (rounded) replaces the x tile
            const int pc = tid % PPR;
            const u32x4 gq = *(const u32x4*)(bias_lds + 6 * C + pc * 8), bq = *(const u32x4*)(bias_lds + 7 * C + pc * 8);
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int rr = (tid + i * THREADS) / PPR;
                const u32x4 o = *(const u32x4*)(ht + rr * XS + pc * 8);
                const u32x4 sh = *(const u32x4*)(sum_lds + rr * XS + pc * 8);   // written by this thread
                u32x4 sm;
                float v[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    sm[k] = H16<T>::pack2(H16<T>::lo(o[k]) + H16<T>::lo(sh[k]), H16<T>::hi(o[k]) + H16<T>::hi(sh[k]));
                    v[2 * k] = H16<T>::lo(sm[k]);
                    v[2 * k + 1] = H16<T>::hi(sm[k]);
                }
                *(u32x4*)(sum_lds + rr * XS + pc * 8) = sm;
                *(u32x4*)(xt + rr * XS + pc * 8) = norm_piece(v, gq, bq, extra.eps);
            }
            __syncthreads();
        }
        if constexpr (HEADM) {
            // ---- the xCPE's Linear on the convolution rows (+ bias), rounded, parked in ht
            bias_from(hacc, bias_lds);
            stage(xt, hacc, 0);
            park(hacc, ht);
            __syncthreads();
            // ---- sum = resid + LayerNorm_cpe(that) (both rounded) to memory; LayerNorm_1(sum) replaces the x tile
            const int pc = tid % PPR;
            const u32x4 gc = *(const u32x4*)(bias_lds + C + pc * 8), bc = *(const u32x4*)(bias_lds + 2 * C + pc * 8);
            const u32x4 g1 = *(const u32x4*)(bias_lds + 3 * C + pc * 8), bb1 = *(const u32x4*)(bias_lds + 4 * C + pc * 8);
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int rr = (tid + i * THREADS) / PPR;
                const u32x4 o = *(const u32x4*)(ht + rr * XS + pc * 8);
                const bool live = row0 + rr < row_end;
                u32x4 sh = {0, 0, 0, 0};
                if (live) sh = *(const u32x4*)(resid + (row0 + rr) * C + pc * 8);
                float v[8];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[2 * k] = H16<T>::lo(o[k]);
                    v[2 * k + 1] = H16<T>::hi(o[k]);
                }
                const u32x4 z = norm_piece(v, gc, bc, extra.eps);
                u32x4 sm;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    sm[k] = H16<T>::pack2(H16<T>::lo(z[k]) + H16<T>::lo(sh[k]), H16<T>::hi(z[k]) + H16<T>::hi(sh[k]));
                    v[2 * k] = H16<T>::lo(sm[k]);
                    v[2 * k + 1] = H16<T>::hi(sm[k]);
                }
                if (live) *(u32x4*)(out + (row0 + rr) * C + pc * 8) = sm;
                *(u32x4*)(xt + rr * XS + pc * 8) = norm_piece(v, g1, bb1, extra.eps1);
            }
            __syncthreads();
            // ---- qkv in three chunks of C outputs: product (+ bias), rounded, through a staging tile to memory in
            // 16-byte pieces. Two staging tiles in turn: a chunk is parked while the one before it is still leaving,
            // and the barrier behind the next park is the one that frees a tile for reuse
#pragma unroll 1
            for (int c = 0; c < 3; ++c) {
                T* tile = (c & 1) ? ht : sum_lds;   // ht was read last by the piece loop above, a barrier ago
                bias_from(hacc, bias_lds + (5 + c) * C);
                stage(xt, hacc, (1 + c) * KU);
                park(hacc, tile);
                __syncthreads();
#pragma unroll
                for (int i = 0; i < PIECES; ++i) {
                    const int rr = (tid + i * THREADS) / PPR;
                    if (row0 + rr < row_end)
                        *(u32x4*)((T*)extra.qkv + (row0 + rr) * (3 * C) + c * C + pc * 8) = *(const u32x4*)(tile + rr * XS + pc * 8);
                }
            }
            // no barrier here: the next pass writes xt (last read before the barrier above), then parks into ht and
            // the other tile only behind barriers of its own that every wave reaches after these stores
            return;
        }
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int rt = 0; rt < RT_; ++rt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[a][rt][v] = 0.f;

#pragma unroll 1   // unrolled, the chunks' loads are hoisted over each other and spill
        for (int c = 0; c < 4; ++c) {
            bias_into(hacc, c);
            stage(xt, hacc, FRONT + 2 * c * KU);
            // hacc[a][rt][v]: hidden unit ch0 + 32 a + 8 (v / 4) + 4 hf + v % 4 of row r0 + 32 rt + col
#pragma unroll
            for (int a = 0; a < MT; ++a)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int hh = ch0 + a * 32 + 8 * g + 4 * hf;
#pragma unroll
                    for (int rt = 0; rt < RT_; ++rt)
                        *(u32x2*)(ht + (r0 + rt * 32 + col) * XS + hh) =
                            (u32x2){gelu_round_pack2<T>(hacc[a][rt][4 * g], hacc[a][rt][4 * g + 1]),
                                    gelu_round_pack2<T>(hacc[a][rt][4 * g + 2], hacc[a][rt][4 * g + 3])};
                }
            __syncthreads();
            stage(ht, acc, FRONT + (2 * c + 1) * KU);
            __syncthreads();
        }

        // ---- fc2 + bias, rounded, parked in LDS; then resid + that in contiguous 16-byte pieces
#pragma unroll
        for (int a = 0; a < MT; ++a)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int cc = ch0 + a * 32 + 8 * g + 4 * hf;
                const u32x2 bb = *(const u32x2*)(bias_lds + 4 * C + cc);
                const float bias[4] = {H16<T>::lo(bb[0]), H16<T>::hi(bb[0]), H16<T>::lo(bb[1]), H16<T>::hi(bb[1])};
#pragma unroll
                for (int rt = 0; rt < RT_; ++rt)
                    *(u32x2*)(ht + (r0 + rt * 32 + col) * XS + cc) =
                        (u32x2){H16<T>::pack2(acc[a][rt][4 * g] + bias[0], acc[a][rt][4 * g + 1] + bias[1]),
                                H16<T>::pack2(acc[a][rt][4 * g + 2] + bias[2], acc[a][rt][4 * g + 3] + bias[3])};
            }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int p = tid + i * THREADS;
            const int rr = p / PPR, pc = p % PPR;
            if (row0 + rr < row_end) {
                const u32x4 o = *(const u32x4*)(ht + rr * XS + pc * 8);
                const u32x4 s = TAIL ? *(const u32x4*)(sum_lds + rr * XS + pc * 8)
                                     : *(const u32x4*)(resid + (row0 + rr) * C + pc * 8);
                u32x4 r;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    r[k] = H16<T>::pack2(H16<T>::lo(o[k]) + H16<T>::lo(s[k]), H16<T>::hi(o[k]) + H16<T>::hi(s[k]));
                *(u32x4*)(out + (row0 + rr) * C + pc * 8) = r;
            }
        }
        // the next pass writes the hidden buffers only after the barrier that follows its x tile load
    };

    // Every work-group does `upw` row groups of 32 WM rows in passes of equal shape: in a round all work-groups take
    // neighbouring tiles of rt row groups (5 = 3 + 2, 4 = 2 + 2), so the rows in flight at any time are one window
    // of the matrix and the last round is as full as the first.
    constexpr int UNIT = 32 * WM;
    int64_t base = 0;   // first row group of the round
    for (int left = upw; left > 0;) {
        const int passes = (left + RTMAX - 1) / RTMAX;
        const int rt = (left + passes - 1) / passes;
        const int64_t row0 = (base + (int64_t)blockIdx.x * rt) * UNIT;
        if (row0 < n) {
            if (RTMAX >= 3 && rt == 3) pass(std::integral_constant<int, (RTMAX >= 3 ? 3 : 1)>{}, row0, n);
            else if (RTMAX >= 2 && rt == 2) pass(std::integral_constant<int, (RTMAX >= 2 ? 2 : 1)>{}, row0, n);
            else pass(std::integral_constant<int, 1>{}, row0, n);
        }
        base += (int64_t)gridDim.x * rt;
        left -= rt;
    }
}

template <typename T, int C, int WM, int WN, int MT, int DEPTH, bool PACKED, int RTMAX, int MODE = MLP_MODE,
          int THREADS = MW_THREADS, int MINW = 2>
int launch_mlp_wide(const void* x, const void* resid, const void* w1, const void* b1, const void* w2, const void* b2,
                    int64_t n, void* out, hipStream_t stream, WideArgs extra = WideArgs{}) {
    constexpr int RMAX = 32 * RTMAX * WM, UNIT = 32 * WM;
    constexpr size_t LDS = ((size_t)(MODE == MLP_MODE ? 2 : 3) * RMAX * (C + MW_PAD) + (MODE == MLP_MODE ? 5 : 8) * C) * sizeof(T);
    static_assert(LDS <= 160 * 1024, "LDS of a CU");
    const size_t lds = LDS;
    auto kern = mlp_wide_kernel<T, C, WM, WN, MT, DEPTH, PACKED, RTMAX, THREADS, MINW, MODE>;
    static LdsGrant grant_configured;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_configured)) return rc_;
    // as many work-groups as the machine holds at a time (MINW waves per SIMD, THREADS / 256 of them from one
    // work-group), each with the same number of row groups
    const int64_t resident = (int64_t)256 * MINW * 256 / THREADS;
    const int64_t units = (n + UNIT - 1) / UNIT;
    const int64_t grid = units < resident ? units : resident;
    const int64_t upw = (units + grid - 1) / grid;
    if (upw > 0x7fffffffLL) return PTV3_EINVAL;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(THREADS), lds, stream,
                       (const T*)x, (const T*)resid, (const T*)w1, (const T*)b1, (const T*)w2, (const T*)b2, n, (int)upw, (T*)out,
                       extra);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

template <bool PACKED>
int mlp_wide_any(const void* x, const void* resid, const void* w1, const void* b1, const void* w2, const void* b2,
                 int dtype, int64_t n, int channels, void* out, hipStream_t stream) {
#define PTV3_MW(T)                                                                                                      \
    do {                                                                                                                \
        if (channels == 128) return launch_mlp_wide<T, 128, 2, 4, 1, 4, PACKED, 3>(x, resid, w1, b1, w2, b2, n, out, stream); \
        if (channels == 256) return launch_mlp_wide<T, 256, 1, 8, 1, 4, PACKED, 3>(x, resid, w1, b1, w2, b2, n, out, stream); \
        if (channels == 512) return launch_mlp_wide<T, 512, 1, 8, 2, 2, PACKED, 2>(x, resid, w1, b1, w2, b2, n, out, stream); \
    } while (0)
    if (dtype == PTV3_F16) PTV3_MW(_Float16);
    if (dtype == PTV3_BF16) PTV3_MW(__bf16);
#undef PTV3_MW
    return PTV3_ESHAPE;
}

int block_tail_wide_any(const void* attn, const void* sum, const void* packed, const void* b1, const void* b2, int dtype,
                        int64_t n, int channels, void* out, hipStream_t stream, WideArgs extra) {
#define PTV3_MW(T)                                                                                                      \
    do {                                                                                                                \
        if (channels == 128)                                                                                            \
            return launch_mlp_wide<T, 128, 2, 4, 1, 4, true, 3, TAIL_MODE>(attn, sum, packed, b1, nullptr, b2, n, out, stream, extra); \
        if (channels == 256)                                                                                            \
            return launch_mlp_wide<T, 256, 1, 8, 1, 4, true, 3, TAIL_MODE>(attn, sum, packed, b1, nullptr, b2, n, out, stream, extra); \
    } while (0)
    if (dtype == PTV3_F16) PTV3_MW(_Float16);
    if (dtype == PTV3_BF16) PTV3_MW(__bf16);
#undef PTV3_MW
    return PTV3_ESHAPE;
}

int block_head_wide_any(const void* conv, const void* shortcut, const void* packed, int dtype, int64_t n, int channels,
                        void* feat, hipStream_t stream, WideArgs args) {
#define PTV3_MW(T)                                                                                                      \
    do {                                                                                                                \
        if (channels == 128)                                                                                            \
            return launch_mlp_wide<T, 128, 2, 4, 1, 4, true, 3, HEAD_MODE>(conv, shortcut, packed, nullptr, nullptr, nullptr, n, feat, stream, args); \
        if (channels == 256)                                                                                            \
            return launch_mlp_wide<T, 256, 1, 8, 1, 4, true, 3, HEAD_MODE>(conv, shortcut, packed, nullptr, nullptr, nullptr, n, feat, stream, args); \
    } while (0)
    if (dtype == PTV3_F16) PTV3_MW(_Float16);
    if (dtype == PTV3_BF16) PTV3_MW(__bf16);
#undef PTV3_MW
    return PTV3_ESHAPE;
}

}  // namespace

// called by ptv3_mlp_fused for channels 128, 256 and 512
int mlp_wide_dispatch(const void* x, const void* resid, const void* w1, const void* b1, const void* w2, const void* b2,
                      int dtype, int64_t n, int channels, void* out, hipStream_t stream) {
    return mlp_wide_any<false>(x, resid, w1, b1, w2, b2, dtype, n, channels, out, stream);
}

extern "C" int ptv3_mlp_pack_weights(const void* w1, const void* w2, int dtype, int channels, void* packed, void* stream_) {
    if (channels != 128 && channels != 256 && channels != 512) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (!w1 || !w2 || !packed) return PTV3_EINVAL;
    const int64_t pieces = (int64_t)channels * channels;
    // both half types are 16-bit patterns here: one instantiation moves either
    hipLaunchKernelGGL(mlp_pack_kernel<_Float16>, dim3((unsigned)ptv3_ceil_div(pieces, 256)), dim3(256), 0,
                       (hipStream_t)stream_, (const _Float16*)w1, (const _Float16*)w2, channels, (_Float16*)packed);
    PTV3_RETURN_LAUNCH();
}

extern "C" int64_t ptv3_mlp_pack_weights_blocks(int channels) {
    if (channels != 128 && channels != 256 && channels != 512) return 0;
    return ptv3_ceil_div((int64_t)channels * channels, 256);
}

extern "C" int ptv3_mlp_pack_weights_batch(const ptv3_mlp_pack_job* jobs, int n_jobs, int64_t n_blocks, void* stream_) {
    if (n_jobs < 0 || n_blocks < 0 || n_blocks > 0x7fffffffLL) return PTV3_EINVAL;
    if (n_jobs == 0 || n_blocks == 0) return PTV3_OK;
    if (!jobs) return PTV3_EINVAL;
    hipLaunchKernelGGL(mlp_pack_batch_kernel, dim3((unsigned)n_blocks), dim3(256), 0, (hipStream_t)stream_, jobs, n_jobs);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_mlp_fused_packed(const void* x, const void* resid, const void* packed, const void* b1, const void* b2,
                                     int dtype, int64_t n, int channels, void* out, void* stream_) {
    if (n < 0) return PTV3_EINVAL;
    if (channels != 128 && channels != 256 && channels != 512) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !resid || !packed || !b1 || !b2 || !out) return PTV3_EINVAL;
    return mlp_wide_any<true>(x, resid, packed, b1, nullptr, b2, dtype, n, channels, out, (hipStream_t)stream_);
}

extern "C" int ptv3_block_tail_wide(const void* attn, const void* shortcut, const void* proj_packed, const void* proj_bias,
                                    const void* ln_weight, const void* ln_bias, float ln_eps, const void* mlp_packed,
                                    const void* b1, const void* b2, int dtype, int64_t n, int channels, void* out,
                                    void* stream_) {
    if (n < 0) return PTV3_EINVAL;
    if (channels != 128 && channels != 256) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!attn || !shortcut || !proj_packed || !proj_bias || !ln_weight || !ln_bias || !mlp_packed || !b1 || !b2 || !out)
        return PTV3_EINVAL;
    return block_tail_wide_any(attn, shortcut, mlp_packed, b1, b2, dtype, n, channels, out, (hipStream_t)stream_,
                               WideArgs{proj_packed, proj_bias, ln_weight, ln_bias, ln_eps, nullptr, nullptr, nullptr, 0.f, nullptr});
}

extern "C" int64_t ptv3_linear_pack_weights_blocks(int channels) {
    if (channels != 128 && channels != 256 && channels != 512) return 0;
    return ptv3_ceil_div((int64_t)channels * channels / 8, 256);
}

extern "C" int ptv3_block_head_wide(const void* conv, const void* shortcut, const void* packed, const void* cpe_bias,
                                    const void* ln_cpe_weight, const void* ln_cpe_bias, float ln_cpe_eps,
                                    const void* ln1_weight, const void* ln1_bias, float ln1_eps, const void* qkv_bias,
                                    int dtype, int64_t n, int channels, void* feat, void* qkv, void* stream_) {
    if (n < 0) return PTV3_EINVAL;
    if (channels != 128 && channels != 256) return PTV3_ESHAPE;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!conv || !shortcut || !packed || !cpe_bias || !ln_cpe_weight || !ln_cpe_bias || !ln1_weight || !ln1_bias ||
        !qkv_bias || !feat || !qkv)
        return PTV3_EINVAL;
    return block_head_wide_any(conv, shortcut, packed, dtype, n, channels, feat, (hipStream_t)stream_,
                               WideArgs{nullptr, cpe_bias, ln_cpe_weight, ln_cpe_bias, ln_cpe_eps, ln1_weight, ln1_bias,
                                        qkv_bias, ln1_eps, qkv});
}
