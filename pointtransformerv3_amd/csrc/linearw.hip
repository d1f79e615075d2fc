// Linear layers of the 256-channel blocks with the weights resident in REGISTERS: out = act(x W^T + b),
// x (n, 256), W (N, 256) as nn.Linear stores it, N a multiple of 256, half precision
// (model.py:541-545 cpe.1, :450 qkv, :487 proj, :510-512 fc1 + GELU at the 16 cm level of the default model).
//
// These layers are MFMA work in principle (38k rows x 256 x 256..1024), but a kernel that fetches an operand
// fragment from LDS for every MFMA is bound by the LDS port (1 KB per 32-cycle MFMA and SIMD = the CU's whole
// 128 B / cycle). Here a work-group takes a tile of 256 output channels and a span of rows; its 8 waves are
// 2 row halves x 4 output-channel quarters, and a wave keeps W[its 64 channels, all 256 inputs] as MFMA operand
// fragments in 128 registers for its whole life (staged once through LDS so that the global reads are whole
// rows). Rows stream through 64 at a time: every row fragment read from LDS meets two weight fragments that are
// already in registers (0.5 KB of LDS traffic per MFMA), and the weights leave L2 once per work-group.
// The rows of a tile go through LDS in 64-channel steps (64 rows x 128 B), double-buffered, one barrier per step,
// software-pipelined by hand: right after the barrier that publishes step s+1 a wave asks for its fragments of
// step s+1 and then issues the eight MFMAs of step s, so the LDS reads run under the matrix work. The rows of the
// next four steps (a whole tile) are in flight in a ring of registers that runs on across tile boundaries.
// Bias and the exact GELU are applied on the accumulators; results are rounded to the storage type once and leave
// as whole row segments (8 rows x 128 B per store) through the wave's own LDS rows.
#include "rowtile.h"

namespace {

constexpr int LW_THREADS = 512;
constexpr int LW_ROWS = 64;
constexpr int LW_KC = 64;
constexpr int LW_XSTRIDE = LW_KC + 8;   // halfs per staged row
constexpr int LW_K = 256, LW_N = 256;
constexpr int LW_WSTRIDE = LW_K + 8;
constexpr int LW_OSTRIDE = 64 + 8;      // halfs per row of a wave's result staging

// What follows the Linear when it is the cpe.1 or proj layer of a 256-channel block (LN = 3, 2; model.py:587-597),
// as in ptv3_linear_ln_fwd: the residual, the LayerNorm(s) and the second output.
template <typename T> struct LwNorm {
    const T *res, *gamma, *beta, *gamma2, *beta2, *shift;
    float eps;
    T* out1;
};

// What the epilogue of a tile needs to know about the lane and its work-group.
template <typename T> struct LwLane {
    T* stage;               // the wave's 32 x 64 staging rows
    const float* b_lds;     // bias [LW_N]
    const float* p_lds;     // LayerNorm parameters [5][LW_N]
    float* ex_lds;          // partial sums of the LayerNorms [4][LW_ROWS][4]
    int c0, row0, col, hf, lane, wave, cout0, nout;
    int64_t n;
};

// acc -> out (and ln.out1) for the 64-row tile that starts at row tile_row0; resv: the residual rows of the wave's
// 32 x 64 block (LN != 0). Contains work-group barriers when LN != 0: every wave calls it the same number of times.
template <typename T, bool GELU, int LN>
__device__ __forceinline__ void lw_epilogue(f32x16 (&acc)[2], const u32x4* resv, const LwLane<T>& L, const LwNorm<T>& ln,
                                            T* out, int64_t tile_row0) {
    constexpr int NT = 2;
    T* stage = L.stage;
    const float *b_lds = L.b_lds, *p_lds = L.p_lds;
    float* ex_lds = L.ex_lds;
    const int c0 = L.c0, row0 = L.row0, col = L.col, hf = L.hf, lane = L.lane, wave = L.wave, cout0 = L.cout0, nout = L.nout;
    const int64_t n = L.n;
    // acc[b][v]: output channel cout0 + c0 + b*32 + 8*(v/4) + 4*hf + v%4 of row row0 + col of the tile
    auto store_rows = [&](T* dst) {   // the wave's staged 32 x 64 block as whole row segments
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int orow = it * 8 + (lane >> 3), opc = lane & 7;
            const u32x4 val = *(const u32x4*)(stage + orow * LW_OSTRIDE + opc * 8);
            int64_t r = tile_row0 + row0 + orow;
            r = r < n ? r : n - 1;
            *(u32x4*)(dst + r * nout + cout0 + c0 + opc * 8) = val;
        }
        asm volatile("" ::: "memory");
    };
    if constexpr (LN == 0) {
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 bb = *(const f32x4*)(b_lds + c0 + b * 32 + 8 * q + 4 * hf);
                float r[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    r[i] = acc[b][4 * q + i] + bb[i];
                    if (GELU) r[i] = gelu_erf(H16<T>::round(r[i]));
                }
                *(u32x2*)(stage + col * LW_OSTRIDE + b * 32 + 8 * q + 4 * hf) =
                    (u32x2){H16<T>::pack2(r[0], r[1]), H16<T>::pack2(r[2], r[3])};
            }
        store_rows(out);
    } else {
        // ---- the residual block through the staging rows into accumulator order
#pragma unroll
        for (int it = 0; it < 4; ++it)
            *(u32x4*)(stage + (it * 8 + (lane >> 3)) * LW_OSTRIDE + (lane & 7) * 8) = resv[it];
        asm volatile("" ::: "memory");
        float val[NT][16];
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f32x4 bb = *(const f32x4*)(b_lds + c0 + b * 32 + 8 * q + 4 * hf);
                const u32x2 rp = *(const u32x2*)(stage + col * LW_OSTRIDE + b * 32 + 8 * q + 4 * hf);
                const float rr[4] = {H16<T>::lo(rp[0]), H16<T>::hi(rp[0]), H16<T>::lo(rp[1]), H16<T>::hi(rp[1])};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float lin = H16<T>::round(acc[b][4 * q + i] + bb[i]);
                    // mode 2: the sum is final here; mode 3: the residual waits in the upper half of the pair
                    val[b][4 * q + i] = LN == 2 ? H16<T>::round(lin + rr[i]) : lin;
                    if (LN == 3) acc[b][4 * q + i] = rr[i];
                }
            }
        asm volatile("" ::: "memory");
        // mean and 1 / std of the wave's row over all 256 channels: slot, slot + 1 of the exchange buffer
        auto row_stats = [&](int slot, float& mean, float& rstd) {
            float sum = 0.f;
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) sum += val[b][v];
            sum += __shfl_xor(sum, 32, PTV3_WAVE);
            float* mine = ex_lds + (slot * LW_ROWS + row0 + col) * 4;
            if (hf == 0) mine[wave & 3] = sum;
            __syncthreads();
            const f32x4 ps = *(const f32x4*)mine;
            mean = (ps[0] + ps[1] + ps[2] + ps[3]) * (1.f / LW_N);
            float dev = 0.f;
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int v = 0; v < 16; ++v) dev += (val[b][v] - mean) * (val[b][v] - mean);
            dev += __shfl_xor(dev, 32, PTV3_WAVE);
            if (hf == 0) mine[LW_ROWS * 4 + (wave & 3)] = dev;
            __syncthreads();
            const f32x4 pd = *(const f32x4*)(mine + LW_ROWS * 4);
            rstd = rsqrtf((pd[0] + pd[1] + pd[2] + pd[3]) * (1.f / LW_N) + ln.eps);
        };
        float mean, rstd;
        if (LN == 3) {   // s = res + LN(lin), every stage rounded
            row_stats(0, mean, rstd);
#pragma unroll
            for (int b = 0; b < NT; ++b)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int c = c0 + b * 32 + 8 * q + 4 * hf;
                    const f32x4 ga = *(const f32x4*)(p_lds + c), be = *(const f32x4*)(p_lds + LW_N + c);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float y = (val[b][4 * q + i] - mean) * rstd * ga[i] + be[i];
                        val[b][4 * q + i] = H16<T>::round(H16<T>::round(y) + acc[b][4 * q + i]);
                    }
                }
        }
        // ---- out0 = s (+ shift), out1 = LN(s) with the second (mode 3) or only (mode 2) parameters
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = c0 + b * 32 + 8 * q + 4 * hf;
                f32x4 sh = {0.f, 0.f, 0.f, 0.f};
                if (LN == 2) sh = *(const f32x4*)(p_lds + 4 * LW_N + c);
                *(u32x2*)(stage + col * LW_OSTRIDE + b * 32 + 8 * q + 4 * hf) =
                    (u32x2){H16<T>::pack2(val[b][4 * q] + sh[0], val[b][4 * q + 1] + sh[1]),
                            H16<T>::pack2(val[b][4 * q + 2] + sh[2], val[b][4 * q + 3] + sh[3])};
            }
        store_rows(out);
        row_stats(2, mean, rstd);
        const float* ga_l = p_lds + (LN == 3 ? 2 * LW_N : 0);
        const float* be_l = p_lds + (LN == 3 ? 3 * LW_N : LW_N);
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = c0 + b * 32 + 8 * q + 4 * hf;
                const f32x4 ga = *(const f32x4*)(ga_l + c), be = *(const f32x4*)(be_l + c);
                float o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (val[b][4 * q + i] - mean) * rstd * ga[i] + be[i];
                *(u32x2*)(stage + col * LW_OSTRIDE + b * 32 + 8 * q + 4 * hf) =
                    (u32x2){H16<T>::pack2(o[0], o[1]), H16<T>::pack2(o[2], o[3])};
            }
        store_rows(ln.out1);
    }
}

// LN = 0: out = act(x W^T + b). LN = 2 / 3 (nout = 256, one tile of output channels, so a work-group holds whole
// rows): modes 2 / 3 of the Linear + LayerNorm kernel on the accumulators, every intermediate rounded where the
// separate kernels store it. A row's 256 channels are spread over the four waves of its row half: the sums of a
// LayerNorm go through LDS (mean first, then the squared deviations), one barrier each.
template <typename T, bool GELU, int LN>
__global__ __launch_bounds__(LW_THREADS, 2) void linear_wide_kernel(
    const T* __restrict__ x, const T* __restrict__ weight, const T* __restrict__ bias, int64_t n, int nout,
    T* __restrict__ out, int span_rows, LwNorm<T> ln) {
    typedef typename H16<T>::v8 v8;
    constexpr int KSTEPS = LW_K / LW_KC;       // 4 = depth of the ring
    constexpr int KS = LW_KC / 16;             // MFMA contraction steps per staged step
    constexpr int NT = 2;
    constexpr int XBUF = LW_ROWS * LW_XSTRIDE;
    static_assert(LW_THREADS == LW_ROWS * (LW_KC / 8), "one 16-byte piece per thread and step");
    extern __shared__ __align__(16) unsigned char lw_smem[];
    T* w_lds = (T*)lw_smem;                       // [LW_N][LW_WSTRIDE], only while the fragments are taken
    T* x_lds = w_lds + LW_N * LW_WSTRIDE;         // [2][LW_ROWS][LW_XSTRIDE]
    float* b_lds = (float*)(x_lds + 2 * XBUF);    // [LW_N]

    const int64_t r0 = (int64_t)blockIdx.x * span_rows;
    if (r0 >= n) return;
    const int64_t r1 = r0 + span_rows < n ? r0 + span_rows : n;
    const int cout0 = blockIdx.y * LW_N;
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int row0 = (wave >> 2) * 32;                 // the wave's first row inside a tile
    const int c0 = (wave & 3) * (NT * 32);             // its first output channel inside the tile
    const int grow = tid >> 3, gpc = tid & 7;          // the row and 16-byte piece this thread fetches

    const int n_tiles = (int)((r1 - r0 + LW_ROWS - 1) / LW_ROWS);
    // rows past the end of the matrix repeat its last row: they compute and store the same values to the same
    // place, so no load or store of the loop is conditional (with a branch around them the wait counts in front
    // of the ring would be those of the path that skips them)
    auto row_ptr = [&](int tile) {
        const int64_t r = r0 + (int64_t)(tile < n_tiles ? tile : n_tiles - 1) * LW_ROWS + grow;
        return x + (r < n ? r : n - 1) * LW_K + gpc * 8;
    };
    const T* ptr_cur = row_ptr(0);
    const T* ptr_nxt = row_ptr(1);
    const T* ptr_nn = row_ptr(2);
    u32x4 ring[KSTEPS];   // ring[r]: the earliest step not yet in LDS whose number is r modulo KSTEPS
#pragma unroll
    for (int j = 0; j < KSTEPS; ++j) ring[j] = *(const u32x4*)(ptr_cur + j * LW_KC);

    // ---- the weights of this tile of output channels: whole rows into LDS, then this wave's fragments into registers
    {
        constexpr int PIECES = LW_N * (LW_K / 8) / LW_THREADS;   // 16 per thread, 8 in flight together
#pragma unroll
        for (int i0 = 0; i0 < PIECES; i0 += 8) {
            u32x4 piece[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * LW_THREADS, co = e / (LW_K / 8), pc = e % (LW_K / 8);
                piece[i] = *(const u32x4*)(weight + (int64_t)(cout0 + co) * LW_K + pc * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * LW_THREADS, co = e / (LW_K / 8), pc = e % (LW_K / 8);
                *(u32x4*)(w_lds + co * LW_WSTRIDE + pc * 8) = piece[i];
            }
        }
        if (tid < LW_N) b_lds[tid] = bias ? (float)bias[cout0 + tid] : 0.f;
    }
    __syncthreads();
    u32x4 wreg[NT][LW_K / 16];
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
        for (int k = 0; k < LW_K / 16; ++k)
            wreg[b][k] = *(const u32x4*)(w_lds + (c0 + b * 32 + col) * LW_WSTRIDE + k * 16 + hf * 8);

    const T* xa = x_lds + (row0 + col) * LW_XSTRIDE + hf * 8;
    T* xw = x_lds + grow * LW_XSTRIDE + gpc * 8;
    asm volatile("" ::"v"(ptr_nn));   // nothing but the ring is in flight when the loop is entered
    // the weight rows in LDS are dead once every wave holds its fragments (the first barrier below): each wave
    // turns its product tiles into row segments there
    T* stage = w_lds + wave * (32 * LW_OSTRIDE);

    // step 0 of the first tile: into buffer 0, its fragments into registers
    *(u32x4*)xw = ring[0];
    ring[0] = *(const u32x4*)ptr_nxt;   // step KSTEPS = step 0 of the second tile
    __syncthreads();
    // behind the staging rows, also where the weights were: the LayerNorm parameters and the waves' partial sums
    float* p_lds = (float*)(w_lds + LW_THREADS / PTV3_WAVE * 32 * LW_OSTRIDE);   // [5][LW_N]
    float* ex_lds = p_lds + 5 * LW_N;                                            // [4][LW_ROWS][4]
    if (LN != 0 && tid < LW_N) {
        p_lds[tid] = (float)ln.gamma[tid];
        p_lds[LW_N + tid] = (float)ln.beta[tid];
        p_lds[2 * LW_N + tid] = LN == 3 ? (float)ln.gamma2[tid] : 0.f;
        p_lds[3 * LW_N + tid] = LN == 3 ? (float)ln.beta2[tid] : 0.f;
        p_lds[4 * LW_N + tid] = (LN == 2 && ln.shift) ? (float)ln.shift[tid] : 0.f;
    }   // published by the first barrier of the loop below
    u32x4 xf[2][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xf[0][ks] = *(const u32x4*)(xa + ks * 16);

    for (int tile = 0; tile < n_tiles; ++tile) {
        const T* ptr_3 = row_ptr(tile + 3);
        u32x4 resv[LN != 0 ? 4 : 1];   // the residual rows of this wave's 32 x 64 block, whole row segments
        if (LN != 0) {
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                int64_t r = r0 + (int64_t)tile * LW_ROWS + row0 + it * 8 + (lane >> 3);
                r = r < n ? r : n - 1;
                resv[it] = *(const u32x4*)(ln.res + r * LW_N + c0 + (lane & 7) * 8);
            }
        }
        f32x16 acc[NT];
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
#pragma unroll
        for (int kc = 0; kc < KSTEPS; ++kc) {
            // publish step kc + 1 (of the next tile when this is the tile's last step) ...
            const int nb = (kc + 1) & 1;
            *(u32x4*)(xw + nb * XBUF) = ring[(kc + 1) % KSTEPS];
            // ... and ask for the step that takes its place in the ring: step kc + 1 of the next tile
            if (kc + 1 < KSTEPS) ring[(kc + 1) % KSTEPS] = *(const u32x4*)(ptr_nxt + (kc + 1) * LW_KC);
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
                    acc[b] = H16<T>::mfma(__builtin_bit_cast(v8, wreg[b][kc * KS + ks]),
                                          __builtin_bit_cast(v8, xf[kc & 1][ks]), acc[b]);
            __builtin_amdgcn_sched_barrier(0);
        }
        const LwLane<T> me = {stage, b_lds, p_lds, ex_lds, c0, row0, col, hf, lane, wave, cout0, nout, n};
        lw_epilogue<T, GELU, LN>(acc, resv, me, ln, out, r0 + (int64_t)tile * LW_ROWS);
        ptr_cur = ptr_nxt;
        ptr_nxt = ptr_nn;
        ptr_nn = ptr_3;
    }
}

// The same layer when a work-group's whole span of rows fits the LDS the weights leave behind (256 outputs and at
// most 192 rows per work-group: up to 49k rows, the 256-channel level of the default model). With three tiles per
// work-group the streaming kernel above never gets past its start-up: a tile of rows is all it has in flight, so it
// runs at the latency of HBM, not its bandwidth. Here every row of the span is asked for before the weights are
// staged (12 x 16 bytes per thread, 96 KB per CU in flight beside the 128 KB of weights), parked in LDS once the
// weights are in registers, and the tiles are then computed without another global load or a barrier per step.
constexpr int RS_TILES = 3;
constexpr int RS_ROWS = RS_TILES * LW_ROWS;        // 192
constexpr int RS_XSTRIDE = LW_K + 8;               // halfs per resident row
constexpr int RS_PIECES = RS_ROWS * (LW_K / 8) / LW_THREADS;   // 16-byte pieces per thread: 12

template <typename T, int LN>
__global__ __launch_bounds__(LW_THREADS, 2) void linear_wide_resident_kernel(
    const T* __restrict__ x, const T* __restrict__ weight, const T* __restrict__ bias, int64_t n, T* __restrict__ out,
    int span_rows, LwNorm<T> ln) {
    typedef typename H16<T>::v8 v8;
    constexpr int NT = 2;
    extern __shared__ __align__(16) unsigned char lw_smem[];
    T* w_lds = (T*)lw_smem;                                   // [LW_N][LW_WSTRIDE], only while the fragments are taken
    float* b_lds = (float*)(w_lds + LW_N * LW_WSTRIDE + 2 * LW_ROWS * LW_XSTRIDE);   // [LW_N], where the other kernel has it
    // after the weights: staging rows of the waves, LayerNorm parameters, partial sums, then the resident rows
    float* p_lds = (float*)(w_lds + LW_THREADS / PTV3_WAVE * 32 * LW_OSTRIDE);        // [5][LW_N]
    float* ex_lds = p_lds + 5 * LW_N;                                                 // [4][LW_ROWS][4]
    T* x_res = (T*)(ex_lds + 4 * LW_ROWS * 4);                                        // [RS_ROWS][RS_XSTRIDE]

    const int64_t r0 = (int64_t)blockIdx.x * span_rows;
    if (r0 >= n) return;
    const int64_t r1 = r0 + span_rows < n ? r0 + span_rows : n;
    const int n_tiles = (int)((r1 - r0 + LW_ROWS - 1) / LW_ROWS);
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int row0 = (wave >> 2) * 32;                 // the wave's first row inside a tile
    const int c0 = (wave & 3) * (NT * 32);             // its first output channel

    // ---- every row of the span: rows past the end of the matrix repeat its last row
    u32x4 xr[RS_PIECES];
#pragma unroll
    for (int i = 0; i < RS_PIECES; ++i) {
        const int e = tid + i * LW_THREADS;
        int64_t r = r0 + e / (LW_K / 8);
        r = r < n ? r : n - 1;
        xr[i] = *(const u32x4*)(x + r * LW_K + (e % (LW_K / 8)) * 8);
    }
    // ---- the weights: whole rows into LDS, then this wave's fragments into registers
    {
        constexpr int PIECES = LW_N * (LW_K / 8) / LW_THREADS;   // 16 per thread, 8 in flight together
#pragma unroll
        for (int i0 = 0; i0 < PIECES; i0 += 8) {
            u32x4 piece[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * LW_THREADS, co = e / (LW_K / 8), pc = e % (LW_K / 8);
                piece[i] = *(const u32x4*)(weight + (int64_t)co * LW_K + pc * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = tid + (i0 + i) * LW_THREADS, co = e / (LW_K / 8), pc = e % (LW_K / 8);
                *(u32x4*)(w_lds + co * LW_WSTRIDE + pc * 8) = piece[i];
            }
        }
        if (tid < LW_N) b_lds[tid] = bias ? (float)bias[tid] : 0.f;
    }
    __syncthreads();
    u32x4 wreg[NT][LW_K / 16];
#pragma unroll
    for (int b = 0; b < NT; ++b)
#pragma unroll
        for (int k = 0; k < LW_K / 16; ++k)
            wreg[b][k] = *(const u32x4*)(w_lds + (c0 + b * 32 + col) * LW_WSTRIDE + k * 16 + hf * 8);
    __syncthreads();   // the weight rows are dead: the rows of the span and the parameters take their place
#pragma unroll
    for (int i = 0; i < RS_PIECES; ++i) {
        const int e = tid + i * LW_THREADS;
        *(u32x4*)(x_res + (e / (LW_K / 8)) * RS_XSTRIDE + (e % (LW_K / 8)) * 8) = xr[i];
    }
    if (LN != 0 && tid < LW_N) {
        p_lds[tid] = (float)ln.gamma[tid];
        p_lds[LW_N + tid] = (float)ln.beta[tid];
        p_lds[2 * LW_N + tid] = LN == 3 ? (float)ln.gamma2[tid] : 0.f;
        p_lds[3 * LW_N + tid] = LN == 3 ? (float)ln.beta2[tid] : 0.f;
        p_lds[4 * LW_N + tid] = (LN == 2 && ln.shift) ? (float)ln.shift[tid] : 0.f;
    }
    T* stage = w_lds + wave * (32 * LW_OSTRIDE);
    const LwLane<T> me = {stage, b_lds, p_lds, ex_lds, c0, row0, col, hf, lane, wave, 0, LW_N, n};
    // the residual rows of the first tile (the wave's 32 x 64 block, whole row segments); a tile ahead from there on
    u32x4 resv[LN != 0 ? 4 : 1], resn[LN != 0 ? 4 : 1];
    auto fetch_res = [&](int tile, u32x4 (&dst)[LN != 0 ? 4 : 1]) {
        if (LN != 0) {
            const int t = tile < n_tiles ? tile : n_tiles - 1;
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                int64_t r = r0 + (int64_t)t * LW_ROWS + row0 + it * 8 + (lane >> 3);
                r = r < n ? r : n - 1;
                dst[it] = *(const u32x4*)(ln.res + r * LW_N + c0 + (lane & 7) * 8);
            }
        }
    };
    fetch_res(0, resv);
    __syncthreads();

    for (int tile = 0; tile < n_tiles; ++tile) {
        fetch_res(tile + 1, resn);
        f32x16 acc[NT];
#pragma unroll
        for (int b = 0; b < NT; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;
        const T* xa = x_res + (tile * LW_ROWS + row0 + col) * RS_XSTRIDE + hf * 8;
#pragma unroll
        for (int k = 0; k < LW_K / 16; ++k) {
            const v8 xf = __builtin_bit_cast(v8, *(const u32x4*)(xa + k * 16));
#pragma unroll
            for (int b = 0; b < NT; ++b) acc[b] = H16<T>::mfma(__builtin_bit_cast(v8, wreg[b][k]), xf, acc[b]);
        }
        lw_epilogue<T, false, LN>(acc, resv, me, ln, out, r0 + (int64_t)tile * LW_ROWS);
        if (LN != 0) {
#pragma unroll
            for (int it = 0; it < 4; ++it) resv[it] = resn[it];
        }
    }
}

template <typename T, bool GELU, int LN = 0>
int launch_linear_wide(const void* x, const void* w, const void* bias, int64_t n, int nout, void* out,
                       hipStream_t stream, LwNorm<T> ln = LwNorm<T>{}) {
    const size_t lds = ((size_t)LW_N * LW_WSTRIDE + 2 * (size_t)LW_ROWS * LW_XSTRIDE) * sizeof(T) + LW_N * sizeof(float);
    static_assert(8 * 32 * LW_OSTRIDE <= LW_N * LW_WSTRIDE, "the waves' staging rows fit where the weights were");
    static_assert((8 * 32 * LW_OSTRIDE) * 2 + (5 * LW_N + 4 * LW_ROWS * 4) * 4 <= LW_N * LW_WSTRIDE * 2,
                  "staging rows, LayerNorm parameters and partial sums fit where the weights were");
    auto kern = linear_wide_kernel<T, GELU, LN>;
    static LdsGrant grant_allowed;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_allowed)) return rc_;
    // one work-group per CU (its registers hold the weights): the 256 CUs are shared out over the tiles of
    // output channels, and every work-group walks an equal span of rows in whole 64-row tiles
    const int col_tiles = nout / LW_N;
    int64_t spans = 256 / col_tiles;
    if (spans < 1) spans = 1;
    int64_t span_rows = ptv3_ceil_div(ptv3_ceil_div(n, spans), LW_ROWS) * LW_ROWS;
    spans = ptv3_ceil_div(n, span_rows);
    if constexpr (!GELU) {
        if (col_tiles == 1 && span_rows <= RS_ROWS) {   // the whole span stays in LDS
            static_assert((8 * 32 * LW_OSTRIDE) * 2 + (5 * LW_N + 4 * LW_ROWS * 4) * 4 + RS_ROWS * RS_XSTRIDE * 2 <=
                              (LW_N * LW_WSTRIDE + 2 * LW_ROWS * LW_XSTRIDE) * 2,
                          "staging rows, parameters, partial sums and the resident rows fit the weights' and tiles' LDS");
            auto rkern = linear_wide_resident_kernel<T, LN>;
            static LdsGrant grant_rallowed;   // per instantiation and device
            if (const int rc_ = ptv3_allow_lds((const void*)rkern, lds, grant_rallowed)) return rc_;
            hipLaunchKernelGGL(rkern, dim3((unsigned)spans), dim3(LW_THREADS), lds, stream, (const T*)x, (const T*)w,
                               (const T*)bias, n, (T*)out, (int)span_rows, ln);
            hipError_t e = hipGetLastError();
            return e == hipSuccess ? PTV3_OK : (int)e;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)spans, (unsigned)col_tiles), dim3(LW_THREADS), lds, stream, (const T*)x,
                       (const T*)w, (const T*)bias, n, nout, (T*)out, (int)span_rows, ln);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}


// ---- Linear layers with long contractions (fc2 of the 256- and 512-channel blocks: 1024 -> 256, 2048 -> 512;
// the 512 -> 1536 qkv): out = resid + x W^T + b, an LDS-tiled GEMM. A work-group of 4 waves owns a
// (MT * 64) x 128 tile of the result; a wave multiplies MT * 32 rows by 64 output channels (MT x 2 accumulator
// tiles: with MT = 4 six operand fragments feed eight MFMAs, 0.75 KB of LDS traffic per MFMA). Both operands
// come through LDS in 64-channel steps, double-buffered, one barrier per step; the pieces of the next two steps
// are in flight in registers. The residual (the stored sum fc2 accumulates onto, model.py:602) is added in fp32
// before the single rounding.
// A 128 x 128 tile moves (128 + 128) x K x 2 bytes out of L2 for 2 x 128 x 128 x K flops, 64 flop per byte: at the
// ~6.5 TB/s the L2s deliver to 256 CUs that is ~410 TFLOP/s, which is what this kernel measures on all three
// shapes (43-48 us; a 256 x 160 tile would move 98 flop per byte). In the default model it takes the two
// 512 -> 1536 qkv layers; fc2 of the wide blocks runs inside the fused MLP kernel.
constexpr int GT_THREADS = 256;
constexpr int GT_N = 128, GT_KC = 64;
constexpr int GT_STRIDE = GT_KC + 8;         // halfs per staged row
constexpr int GT_OSTRIDE = 64 + 8;           // halfs per row of a wave's result staging
constexpr int GT_DEPTH = 2;

template <typename T, int MT>
__global__ __launch_bounds__(GT_THREADS, 2) void linear_gemm_kernel(
    const T* __restrict__ x, const T* __restrict__ weight, const T* __restrict__ bias, const T* resid,
    int64_t n, int k, int nout, T* out) {   // resid may be out itself (fc2 accumulating onto the stored sum)
    typedef typename H16<T>::v8 v8;
    constexpr int GT_M = MT * 64;
    constexpr int XBUF = GT_M * GT_STRIDE, WBUF = GT_N * GT_STRIDE;
    constexpr int PPR = GT_KC / 8;                                           // 16-byte pieces per staged row
    constexpr int RPS = GT_THREADS / PPR;                                    // rows staged per pass of the work-group
    constexpr int XP = GT_M / RPS, WP = GT_N / RPS;                          // pieces per thread and step
    extern __shared__ __align__(16) unsigned char gt_smem[];
    T* lds = (T*)gt_smem;                                // [2 buffers][x tile | w tile]
    static_assert(4 * 32 * GT_OSTRIDE <= 2 * (XBUF + WBUF), "the waves' staging rows fit where the operands were");
    static_assert(GT_M % RPS == 0 && GT_N % RPS == 0, "whole passes");
    const int tid = threadIdx.x, wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    const int col = lane & 31, hf = lane >> 5;
    const int64_t m0 = (int64_t)blockIdx.x * GT_M;
    const int n0 = blockIdx.y * GT_N;
    const int wr = (wave >> 1) * (MT * 32), wc = (wave & 1) * 64;   // the wave's rows and output channels inside the tile
    // staging: thread -> row tid / PPR (+ RPS i), 16-byte piece tid % PPR; rows past the end repeat the last row
    const int srow = tid / PPR, spc = tid % PPR;
    const T* xp[XP];
    const T* wp[WP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int64_t r = m0 + srow + RPS * i;
        xp[i] = x + (r < n ? r : n - 1) * k + spc * 8;
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) wp[i] = weight + (int64_t)(n0 + srow + RPS * i) * k + spc * 8;
    const int steps = k / GT_KC;
    u32x4 xr[GT_DEPTH][XP], wr4[GT_DEPTH][WP];
#pragma unroll
    for (int d = 0; d < GT_DEPTH; ++d) {
        const int sd = d < steps ? d : steps - 1;
#pragma unroll
        for (int i = 0; i < XP; ++i) xr[d][i] = *(const u32x4*)(xp[i] + sd * GT_KC);
#pragma unroll
        for (int i = 0; i < WP; ++i) wr4[d][i] = *(const u32x4*)(wp[i] + sd * GT_KC);
    }
    f32x16 acc[MT][2];
#pragma unroll
    for (int a = 0; a < MT; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;
    // nothing in flight when the loop is entered: the wait-count bookkeeping of a loop is the union of its entry
    // and its back edge, and with loads pending at entry it settled for draining everything once per trip
#pragma unroll
    for (int d = 0; d < GT_DEPTH; ++d) {
#pragma unroll
        for (int i = 0; i < XP; ++i) asm volatile("" ::"v"(xr[d][i]));
#pragma unroll
        for (int i = 0; i < WP; ++i) asm volatile("" ::"v"(wr4[d][i]));
    }
    // two steps per trip so that the ring position and the buffer are compile-time constants (steps is even)
    for (int s0 = 0; s0 < steps; s0 += 2) {
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            const int s = s0 + d;
            T* xb = lds + d * (XBUF + WBUF);
            T* wb = xb + XBUF;
#pragma unroll
            for (int i = 0; i < XP; ++i) *(u32x4*)(xb + (srow + RPS * i) * GT_STRIDE + spc * 8) = xr[d][i];
#pragma unroll
            for (int i = 0; i < WP; ++i) *(u32x4*)(wb + (srow + RPS * i) * GT_STRIDE + spc * 8) = wr4[d][i];
            const int sn = s + GT_DEPTH < steps ? s + GT_DEPTH : steps - 1;   // past the end: a valid address, never used
#pragma unroll
            for (int i = 0; i < XP; ++i) xr[d][i] = *(const u32x4*)(xp[i] + sn * GT_KC);
#pragma unroll
            for (int i = 0; i < WP; ++i) wr4[d][i] = *(const u32x4*)(wp[i] + sn * GT_KC);
            __syncthreads();
#pragma unroll
            for (int ks = 0; ks < GT_KC / 16; ++ks) {
                u32x4 xf[MT], wf[2];
#pragma unroll
                for (int a = 0; a < MT; ++a) xf[a] = *(const u32x4*)(xb + (wr + a * 32 + col) * GT_STRIDE + ks * 16 + hf * 8);
#pragma unroll
                for (int b = 0; b < 2; ++b) wf[b] = *(const u32x4*)(wb + (wc + b * 32 + col) * GT_STRIDE + ks * 16 + hf * 8);
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int a = 0; a < MT; ++a)
                        acc[a][b] = H16<T>::mfma(__builtin_bit_cast(v8, wf[b]), __builtin_bit_cast(v8, xf[a]), acc[a][b]);
            }
        }
    }
    __syncthreads();   // every wave is through with the operand tiles: their room takes the results
    // acc[a][b][v]: output channel n0 + wc + b*32 + 8*(v/4) + 4*hf + v%4 of row m0 + wr + a*32 + col
    T* stage = lds + wave * (32 * GT_OSTRIDE);
    // bias of the lane's output channels: 4 consecutive ones per (b, q)
    float bb[2][4][4];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = n0 + wc + b * 32 + 8 * q + 4 * hf;
            u32x2 raw = {0u, 0u};
            if (bias) raw = *(const u32x2*)(bias + c);
            bb[b][q][0] = H16<T>::lo(raw[0]); bb[b][q][1] = H16<T>::hi(raw[0]);
            bb[b][q][2] = H16<T>::lo(raw[1]); bb[b][q][3] = H16<T>::hi(raw[1]);
        }
#pragma unroll
    for (int a = 0; a < MT; ++a) {
        // the residual rows come in as whole row segments (8 rows x 128 B per load) and pass through the wave's
        // LDS rows into the accumulators' layout: one 8-byte piece per lane read straight from memory would touch
        // 32 cache lines per instruction
        if (resid) {
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int orow = it * 8 + (lane >> 3), opc = lane & 7;
                const int64_t row = m0 + wr + a * 32 + orow;
                u32x4 old = {0u, 0u, 0u, 0u};
                if (row < n) old = *(const u32x4*)(resid + row * nout + n0 + wc + opc * 8);
                *(u32x4*)(stage + orow * GT_OSTRIDE + opc * 8) = old;
            }
            asm volatile("" ::: "memory");
        }
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                T* at = stage + col * GT_OSTRIDE + b * 32 + 8 * q + 4 * hf;
                float r[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) r[i] = acc[a][b][4 * q + i] + bb[b][q][i];
                if (resid) {
                    const u32x2 old = *(const u32x2*)at;
                    r[0] += H16<T>::lo(old[0]); r[1] += H16<T>::hi(old[0]);
                    r[2] += H16<T>::lo(old[1]); r[3] += H16<T>::hi(old[1]);
                }
                *(u32x2*)at = (u32x2){H16<T>::pack2(r[0], r[1]), H16<T>::pack2(r[2], r[3])};
            }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int orow = it * 8 + (lane >> 3), opc = lane & 7;
            const u32x4 val = *(const u32x4*)(stage + orow * GT_OSTRIDE + opc * 8);
            const int64_t row = m0 + wr + a * 32 + orow;
            if (row < n) *(u32x4*)(out + row * nout + n0 + wc + opc * 8) = val;
        }
        asm volatile("" ::: "memory");
    }
}

template <typename T, int MT>
int launch_linear_gemm_mt(const void* x, const void* w, const void* bias, const void* resid, int64_t n, int k, int nout,
                          void* out, hipStream_t stream) {
    const size_t lds = 2 * (size_t)(MT * 64 + GT_N) * GT_STRIDE * sizeof(T);
    auto kern = linear_gemm_kernel<T, MT>;
    static LdsGrant grant_allowed;   // per instantiation and device
    if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant_allowed)) return rc_;
    hipLaunchKernelGGL(kern, dim3((unsigned)ptv3_ceil_div(n, MT * 64), (unsigned)(nout / GT_N)), dim3(GT_THREADS), lds,
                       stream, (const T*)x, (const T*)w, (const T*)bias, (const T*)resid, n, k, nout, (T*)out);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PTV3_OK : (int)e;
}

template <typename T>
int launch_linear_gemm(const void* x, const void* w, const void* bias, const void* resid, int64_t n, int k, int nout,
                       void* out, hipStream_t stream) {
    // 128 x 128 tiles: 256-row tiles would halve the weight traffic per row but need more registers than two
    // work-groups per CU leave, and on these shapes give fewer work-groups than there are CUs
    return launch_linear_gemm_mt<T, 2>(x, w, bias, resid, n, k, nout, out, stream);
}

}  // namespace

// called by ptv3_linear_ln_fwd for 256 channels (modes 2 and 3)
int linear_wide_ln_dispatch(const void* x, const void* w, const void* bias, const void* res, const void* gamma,
                            const void* beta, const void* gamma2, const void* beta2, const void* shift, int dtype,
                            int64_t n, int mode, float eps, void* out0, void* out1, hipStream_t stream) {
#define PTV3_LWLN(T, M)                                                                                         \
    return launch_linear_wide<T, false, M>(x, w, bias, n, LW_N, out0, stream,                                   \
                                           LwNorm<T>{(const T*)res, (const T*)gamma, (const T*)beta, (const T*)gamma2, \
                                                     (const T*)beta2, (const T*)shift, eps, (T*)out1})
    if (dtype == PTV3_F16) {
        if (mode == 2) PTV3_LWLN(_Float16, 2);
        PTV3_LWLN(_Float16, 3);
    }
    if (mode == 2) PTV3_LWLN(__bf16, 2);
    PTV3_LWLN(__bf16, 3);
#undef PTV3_LWLN
}

extern "C" int ptv3_linear_wide_fwd(const void* x, const void* w, const void* bias, int dtype, int64_t n, int k,
                                    int nout, int gelu, void* out, void* stream_) {
    if (n < 0 || k < 1 || nout < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (k != LW_K || nout % LW_N != 0) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16)
        return gelu ? launch_linear_wide<_Float16, true>(x, w, bias, n, nout, out, stream)
                    : launch_linear_wide<_Float16, false>(x, w, bias, n, nout, out, stream);
    return gelu ? launch_linear_wide<__bf16, true>(x, w, bias, n, nout, out, stream)
                : launch_linear_wide<__bf16, false>(x, w, bias, n, nout, out, stream);
}

extern "C" int ptv3_linear_gemm_fwd(const void* x, const void* w, const void* bias, const void* resid, int dtype,
                                    int64_t n, int k, int nout, void* out, void* stream_) {
    if (n < 0 || k < 1 || nout < 1) return PTV3_EINVAL;
    if (dtype != PTV3_F16 && dtype != PTV3_BF16) return PTV3_ESHAPE;
    if (k % (2 * GT_KC) != 0 || nout % GT_N != 0) return PTV3_ESHAPE;
    if (n == 0) return PTV3_OK;
    if (!x || !w || !out) return PTV3_EINVAL;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == PTV3_F16) return launch_linear_gemm<_Float16>(x, w, bias, resid, n, k, nout, out, stream);
    return launch_linear_gemm<__bf16>(x, w, bias, resid, n, k, nout, out, stream);
}
