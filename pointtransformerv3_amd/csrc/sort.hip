// Batched LSD radix argsort of (k, n) int64 curve codes, with the inverse permutation
// produced by the last pass.
//
// Replaces torch.argsort + scatter_ at model.py:119-126 and :667-674 of the reference.
// Only the significant low bits are sorted (3*depth + batch bits, e.g. 29 instead of 64),
// 8 bits per pass; all k rows share every launch (blockIdx.y = row). Between passes a point
// travels as (key, 32-bit index) with the key cut to 32 bits whenever the significant bits fit
// (every released configuration at its adaptive depth): 8 bytes in and 8 out per pass instead of 12.
// A pass is
//   tile_hist  : per-tile digit histogram (LDS atomics)
//   scatter    : stable rank inside the tile by wave-level digit matching; the tile is put in
//                digit order in LDS first, so that the global writes of one digit are contiguous
//                runs instead of 8192 scattered stores. Where a row has at most FUSED_TILES tiles
//                (half a million points: what the model sorts) every work-group finds the global
//                start of its runs itself, by summing the histograms of the tiles in front of it
//                (a few hundred KB out of L2) -- two launches per pass, no scan kernel, no
//                zeroing kernel.
//   tile_scan  : (longer rows only) global start of every (tile, digit) run: exclusive scan of
//                the 256 digit totals, then per digit a running sum over the tiles; 16 blocks per
//                row, 16 digits each; the digit totals come from global atomics of tile_hist.
// int64 order / inverse appear only in the last pass.
#include "common.h"

namespace {

constexpr int RADIX = 256;
constexpr int SORT_THREADS = 512;
constexpr int SORT_WAVES = SORT_THREADS / PTV3_WAVE;
constexpr int SORT_ITEMS = 16;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;   // 8192 keys
constexpr int MAX_PASSES = 8;
constexpr int FUSED_TILES = 64;   // rows of up to 524,288 keys take the two-launch pass

__global__ __launch_bounds__(256) void zero_totals_kernel(uint32_t* __restrict__ totals, int count) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) totals[i] = 0u;
}

// KT: type of the keys read (int64_t codes in the first pass, uint32_t / uint64_t afterwards)
template <typename KT>
__global__ __launch_bounds__(SORT_THREADS) void tile_hist_kernel(
    const KT* __restrict__ keys, int64_t n, int shift, uint32_t* __restrict__ tile_hist,
    int tiles, uint32_t* __restrict__ totals) {
    __shared__ uint32_t hist[RADIX];
    const int row = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
    if (tid < RADIX) hist[tid] = 0;
    __syncthreads();
    const int64_t base = (int64_t)tile * SORT_TILE;
    const KT* src = keys + (int64_t)row * n;
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int64_t i = base + j * SORT_THREADS + tid;
        if (i < n) atomicAdd(&hist[(uint32_t)((uint64_t)src[i] >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid < RADIX) {
        const uint32_t c = hist[tid];
        tile_hist[((int64_t)row * tiles + tile) * RADIX + tid] = c;
        if (totals && c) atomicAdd(&totals[row * RADIX + tid], c);
    }
}

// grid (k, 16): block (row, dg) turns the counts of digits 16 dg .. 16 dg + 15 into global starts.
// Thread (slice, d) owns one digit over one sixteenth of the tiles.
constexpr int SCAN_SLICES = 16, SCAN_DIGITS = RADIX / SCAN_SLICES;
__global__ __launch_bounds__(RADIX) void tile_scan_kernel(uint32_t* __restrict__ tile_hist, int tiles,
                                                          const uint32_t* __restrict__ totals) {
    __shared__ uint32_t base[RADIX];
    __shared__ uint32_t part[SCAN_SLICES][SCAN_DIGITS];
    constexpr int CH = 8;
    const int row = blockIdx.x, dg = blockIdx.y, tid = threadIdx.x;
    // exclusive scan of the row's digit totals (Hillis-Steele over 256 threads)
    const uint32_t mine = totals[row * RADIX + tid];
    base[tid] = mine;
    __syncthreads();
    for (int off = 1; off < RADIX; off <<= 1) {
        const uint32_t v = tid >= off ? base[tid - off] : 0u;
        __syncthreads();
        base[tid] += v;
        __syncthreads();
    }
    const int d = tid % SCAN_DIGITS, slice = tid / SCAN_DIGITS;
    const int digit = dg * SCAN_DIGITS + d;
    const int per = (tiles + SCAN_SLICES - 1) / SCAN_SLICES;
    const int t_lo = min(slice * per, tiles), t_hi = min(t_lo + per, tiles);
    uint32_t* h = tile_hist + (int64_t)row * tiles * RADIX + digit;
    uint32_t sum = 0;
    for (int t0 = t_lo; t0 < t_hi; t0 += CH) {
        uint32_t c[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) c[j] = (t0 + j < t_hi) ? h[(int64_t)(t0 + j) * RADIX] : 0u;
#pragma unroll
        for (int j = 0; j < CH; ++j) sum += c[j];
    }
    part[slice][d] = sum;
    __syncthreads();
    uint32_t run = base[digit] - totals[row * RADIX + digit];   // exclusive digit base
    for (int k = 0; k < slice; ++k) run += part[k][d];
    for (int t0 = t_lo; t0 < t_hi; t0 += CH) {
        uint32_t c[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) c[j] = (t0 + j < t_hi) ? h[(int64_t)(t0 + j) * RADIX] : 0u;
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (t0 + j < t_hi) h[(int64_t)(t0 + j) * RADIX] = run;
            run += c[j];
        }
    }
}

// KI: type of the keys read (int64_t codes in the first pass), KO: type of the keys kept between passes.
// FUSED: tile_off holds the raw per-tile histograms and this work-group derives its global starts from them;
// otherwise tile_off already holds the global start of every (tile, digit) run.
template <typename KI, typename KO, bool FIRST, bool LAST, bool FUSED>
__global__ __launch_bounds__(SORT_THREADS) void scatter_kernel(
    const KI* __restrict__ keys_in, const int32_t* __restrict__ idx_in, int64_t n, int shift,
    const uint32_t* __restrict__ tile_off, int tiles, KO* __restrict__ keys_out,
    int32_t* __restrict__ idx_out, int64_t* __restrict__ order, int64_t* __restrict__ inverse) {
    __shared__ uint32_t whist[SORT_WAVES][RADIX];   // per wave and digit: count, then start inside the sorted tile
    __shared__ uint32_t gdelta[RADIX];              // global start of the digit's run minus its start inside the tile
    __shared__ uint32_t wsum[SORT_WAVES];
    __shared__ uint32_t dbase[RADIX];               // FUSED: inclusive scan of the row's digit totals
    extern __shared__ __align__(16) unsigned char sort_smem[];   // the tile in digit order: keys, then indices
    KO* skey = (KO*)sort_smem;
    int32_t* sidx = (int32_t*)(sort_smem + sizeof(KO) * SORT_TILE);
    const int row = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    for (int e = tid; e < SORT_WAVES * RADIX; e += SORT_THREADS) (&whist[0][0])[e] = 0;
    __syncthreads();

    const int64_t rbase = (int64_t)row * n;
    const int64_t tbase = (int64_t)tile * SORT_TILE;
    const int64_t wbase = tbase + (int64_t)wave * (PTV3_WAVE * SORT_ITEMS);
    KO key[SORT_ITEMS];
    int32_t idx[SORT_ITEMS];
    uint32_t rank[SORT_ITEMS];
    const uint64_t below = (1ull << lane) - 1ull;

#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int64_t i = wbase + j * PTV3_WAVE + lane;
        const bool valid = i < n;
        key[j] = valid ? (KO)keys_in[rbase + i] : (KO)0;
        idx[j] = FIRST ? (int32_t)i : (valid ? idx_in[rbase + i] : 0);
    }
    // FUSED: the global start of this tile's run of digit `tid` = (keys of smaller digits in the whole row)
    // + (keys of this digit in the tiles in front); the loads are issued here and summed below, behind the ranking
    uint32_t total_d = 0, before_d = 0;
    if (FUSED && tid < RADIX) {
        const uint32_t* h = tile_off + (int64_t)row * tiles * RADIX + tid;
        constexpr int CH = 8;
        for (int t0 = 0; t0 < tiles; t0 += CH) {
            uint32_t c[CH];
#pragma unroll
            for (int j = 0; j < CH; ++j) c[j] = (t0 + j < tiles) ? h[(int64_t)(t0 + j) * RADIX] : 0u;
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                total_d += c[j];
                if (t0 + j < tile) before_d += c[j];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const bool valid = wbase + j * PTV3_WAVE + lane < n;
        const uint32_t digit = (uint32_t)((uint64_t)key[j] >> shift) & 255u;
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (digit >> b) & 1u;
            const uint64_t bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        // peers: valid lanes of this wave whose digit equals mine (meaningless if !valid)
        const int leader = __ffsll((unsigned long long)peers) - 1;
        uint32_t pre = 0;
        if (valid && lane == leader) pre = atomicAdd(&whist[wave][digit], (uint32_t)__popcll(peers));
        pre = __shfl(pre, leader < 0 ? 0 : leader, PTV3_WAVE);
        rank[j] = pre + (uint32_t)__popcll(peers & below);
    }
    if (FUSED && tid < RADIX) dbase[tid] = total_d;
    __syncthreads();
    if (FUSED) {
        // inclusive scan of the digit totals over the 256 digits
        for (int off = 1; off < RADIX; off <<= 1) {
            const uint32_t v = (tid < RADIX && tid >= off) ? dbase[tid - off] : 0u;
            __syncthreads();
            if (tid < RADIX) dbase[tid] += v;
            __syncthreads();
        }
    }
    // digit `tid` (the first 256 threads = four whole waves): its start inside the sorted tile (exclusive scan of
    // the tile histogram over the digits), the starts of each wave's run of it, and where the run goes globally
    uint32_t c[SORT_WAVES], total = 0, x = 0;
    if (tid < RADIX) {
#pragma unroll
        for (int w = 0; w < SORT_WAVES; ++w) { c[w] = whist[w][tid]; total += c[w]; }
        x = total;
#pragma unroll
        for (int off = 1; off < PTV3_WAVE; off <<= 1) {
            const uint32_t y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        if (lane == PTV3_WAVE - 1) wsum[wave] = x;
    }
    __syncthreads();
    if (tid < RADIX) {
        uint32_t start = x - total;
        for (int w = 0; w < wave; ++w) start += wsum[w];
        const uint32_t gstart = FUSED ? dbase[tid] - total_d + before_d
                                      : tile_off[((int64_t)row * tiles + tile) * RADIX + tid];
        gdelta[tid] = gstart - start;
#pragma unroll
        for (int w = 0; w < SORT_WAVES; ++w) { whist[w][tid] = start; start += c[w]; }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        if (wbase + j * PTV3_WAVE + lane < n) {
            const uint32_t digit = (uint32_t)((uint64_t)key[j] >> shift) & 255u;
            const uint32_t lp = whist[wave][digit] + rank[j];
            skey[lp] = key[j];
            sidx[lp] = idx[j];
        }
    }
    __syncthreads();
    const int count = (int)(n - tbase < SORT_TILE ? n - tbase : SORT_TILE);
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int lp = j * SORT_THREADS + tid;
        if (lp < count) {
            const KO kv = skey[lp];
            const int32_t iv = sidx[lp];
            const uint32_t digit = (uint32_t)((uint64_t)kv >> shift) & 255u;
            const int64_t pos = (int64_t)(uint32_t)(gdelta[digit] + (uint32_t)lp);
            if (LAST) {
                order[rbase + pos] = iv;
                inverse[rbase + iv] = pos;
            } else {
                keys_out[rbase + pos] = kv;
                idx_out[rbase + pos] = iv;
            }
        }
    }
}

struct SortWs {
    void* keys[2];      // (k, n) of uint64_t (or uint32_t: the same room is reserved either way)
    int32_t* idx[2];
    uint32_t* tile_hist;
    uint32_t* totals;   // [MAX_PASSES][k][RADIX]
    size_t bytes;
};

SortWs carve(void* base, int64_t n, int k) {
    SortWs w;
    const int64_t tiles = ptv3_ceil_div(n > 0 ? n : 1, SORT_TILE);
    size_t off = 0;
    char* p = (char*)base;
    for (int i = 0; i < 2; ++i) {
        w.keys[i] = (void*)(p + off);
        off += ptv3_align256((size_t)k * n * sizeof(int64_t));
    }
    for (int i = 0; i < 2; ++i) {
        w.idx[i] = (int32_t*)(p + off);
        off += ptv3_align256((size_t)k * n * sizeof(int32_t));
    }
    w.tile_hist = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)k * tiles * RADIX * sizeof(uint32_t));
    w.totals = (uint32_t*)(p + off);
    off += ptv3_align256((size_t)MAX_PASSES * k * RADIX * sizeof(uint32_t));
    w.bytes = off;
    return w;
}

template <typename KO>
int run_passes(const int64_t* code, int64_t n, int k, int passes, int64_t* order, int64_t* inverse, const SortWs& w,
                hipStream_t stream) {
    const int tiles = (int)ptv3_ceil_div(n, SORT_TILE);
    const bool fused = tiles <= FUSED_TILES;
    const size_t lds = (sizeof(KO) + sizeof(int32_t)) * SORT_TILE;
    const dim3 grid((unsigned)tiles, (unsigned)k), block(SORT_THREADS);
    if (!fused) {
        const int n_totals = passes * k * RADIX;
        hipLaunchKernelGGL(zero_totals_kernel, dim3((unsigned)ptv3_ceil_div(n_totals, 256)), dim3(256), 0, stream,
                           w.totals, n_totals);
    }
    const KO* kin = nullptr;
    const int32_t* iin = nullptr;
    for (int p = 0; p < passes; ++p) {
        const int shift = 8 * p;
        const bool first = (p == 0), last = (p == passes - 1);
        KO* kout = (KO*)w.keys[p & 1];
        int32_t* iout = w.idx[p & 1];
        uint32_t* totals = fused ? nullptr : w.totals + (size_t)p * k * RADIX;
        if (first)
            hipLaunchKernelGGL(tile_hist_kernel<int64_t>, grid, block, 0, stream, code, n, shift, w.tile_hist, tiles, totals);
        else
            hipLaunchKernelGGL(tile_hist_kernel<KO>, grid, block, 0, stream, kin, n, shift, w.tile_hist, tiles, totals);
        if (!fused)
            hipLaunchKernelGGL(tile_scan_kernel, dim3((unsigned)k, SCAN_SLICES), dim3(RADIX), 0, stream, w.tile_hist, tiles,
                               (const uint32_t*)totals);
#define PTV3_SCATTER(KI, IN, F, L, U)                                                                       \
    do {                                                                                                    \
        auto kern = scatter_kernel<KI, KO, F, L, U>;                                                        \
        static LdsGrant grant; /* per instantiation and device: the tile needs more than the default 64 KB */ \
        if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant)) return rc_;                      \
        hipLaunchKernelGGL(kern, grid, block, lds, stream, IN, iin, n, shift, (const uint32_t*)w.tile_hist, tiles, kout, \
                           iout, order, inverse);                                                           \
    } while (0)
#define PTV3_SCATTER_FL(U)                                                 \
    do {                                                                   \
        if (first && last) PTV3_SCATTER(int64_t, code, true, true, U);     \
        else if (first) PTV3_SCATTER(int64_t, code, true, false, U);       \
        else if (last) PTV3_SCATTER(KO, kin, false, true, U);              \
        else PTV3_SCATTER(KO, kin, false, false, U);                       \
    } while (0)
        if (fused) PTV3_SCATTER_FL(true);
        else PTV3_SCATTER_FL(false);
#undef PTV3_SCATTER_FL
#undef PTV3_SCATTER
        kin = kout;
        iin = iout;
    }
    return PTV3_OK;
}

}  // namespace

extern "C" size_t ptv3_argsort_workspace_bytes(int64_t n, int k) {
    if (n < 0 || k < 1) return 0;
    return carve(nullptr, n, k).bytes;
}

extern "C" int ptv3_argsort(const int64_t* code, int64_t n, int k, int key_bits, int64_t* order,
                            int64_t* inverse, void* workspace, size_t workspace_bytes,
                            void* stream_) {
    if (n < 0 || k < 1 || k > 65535 || n >= (1ll << 31)) return PTV3_EINVAL;
    if (key_bits < 1 || key_bits > 63) return PTV3_EDEPTH;
    if (n == 0) return PTV3_OK;
    if (!code || !order || !inverse || !workspace) return PTV3_EINVAL;
    SortWs w = carve(workspace, n, k);
    if (workspace_bytes < w.bytes) return PTV3_EWORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    const int passes = (key_bits + 7) / 8;
    // the bits above key_bits are equal across a row (the contract), so cutting the keys to 32 bits keeps the order
    const int rc = key_bits <= 32 ? run_passes<uint32_t>(code, n, k, passes, order, inverse, w, stream)
                                  : run_passes<uint64_t>(code, n, k, passes, order, inverse, w, stream);
    if (rc != PTV3_OK) return rc;
    PTV3_RETURN_LAUNCH();
}
