// Batched LSD radix argsort of (k, n) int64 curve codes, with the inverse permutation
// produced by the last pass.
//
// Replaces torch.argsort + scatter_ at model.py:119-126 and :667-674 of the reference.
// Only the significant low bits are sorted (3*depth + batch bits, e.g. 29 instead of 64),
// 8 bits per pass; all k rows share every launch (blockIdx.y = row). Between passes a point
// travels as (key, 32-bit index) with the key cut to 32 bits whenever the significant bits fit
// (every released configuration at its adaptive depth): 8 bytes in and 8 out per pass instead of 12.
// The keys are read once per pass and once up front:
//   digit_totals : one pass over the codes counts, for EVERY pass at once, how many keys of a row have each
//                  digit value (LDS histograms, one global atomic per work-group, digit and pass). Their prefix
//                  sums are where each digit's keys start in the sorted row.
//   scatter      : one launch per pass. A work-group ranks its tile of 8192 keys (stable, by wave-level digit
//                  matching), publishes the tile's digit counts, and adds up the counts of the tiles in front of
//                  it by looking back over what they published (a 64-bit word per tile and digit: status in the
//                  upper half, count in the lower, written and read with device-scope atomics, so that the pair
//                  is seen whole and seen across the XCDs' L2s). A tile that has finished its own sum publishes the
//                  inclusive sum, and the walk of a later tile stops there: in a long row a tile reads the few
//                  tiles that run beside it, not all that came before. Work-groups are dispatched in launch
//                  order, so everything a tile waits for is already running or done; the wait is bounded all the
//                  same (a flag in the workspace is raised and the sort goes on, wrong, rather than hang).
//                  The tile is put in digit order in LDS first, so that the global writes of one digit are
//                  contiguous runs instead of 8192 scattered stores.
// Status values grow with the pass number (2 pass + 1: counts, 2 pass + 2: inclusive sums), so the words are
// cleared once per sort, not once per pass. int64 order / inverse appear only in the last pass.
#include "common.h"

namespace {

constexpr int RADIX = 256;
constexpr int SORT_THREADS = 512;
constexpr int SORT_WAVES = SORT_THREADS / PTV3_WAVE;
constexpr int SORT_ITEMS = 16;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;   // 8192 keys
constexpr int MAX_PASSES = 8;
constexpr int SPIN_LIMIT = 1 << 20;   // look-back polls before a tile gives up waiting (seconds; never reached)

__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* __restrict__ words, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) words[i] = 0u;
}

// totals[pass][row][digit] += keys of the tile with that digit in that pass, all passes from one read
__global__ __launch_bounds__(SORT_THREADS) void digit_totals_kernel(const int64_t* __restrict__ keys, int64_t n, int passes,
                                                                    int k, uint32_t* __restrict__ totals) {
    __shared__ uint32_t hist[MAX_PASSES][RADIX];
    const int row = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
    for (int e = tid; e < passes * RADIX; e += SORT_THREADS) (&hist[0][0])[e] = 0;
    __syncthreads();
    const int64_t base = (int64_t)tile * SORT_TILE;
    const int64_t* src = keys + (int64_t)row * n;
#pragma unroll 4
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int64_t i = base + j * SORT_THREADS + tid;
        if (i < n) {
            const uint64_t key = (uint64_t)src[i];
            for (int p = 0; p < passes; ++p) atomicAdd(&hist[p][(uint32_t)(key >> (8 * p)) & 255u], 1u);
        }
    }
    __syncthreads();
    for (int e = tid; e < passes * RADIX; e += SORT_THREADS) {
        const uint32_t c = (&hist[0][0])[e];
        if (c) atomicAdd(&totals[((int64_t)(e / RADIX) * k + row) * RADIX + e % RADIX], c);
    }
}

__device__ __forceinline__ uint64_t look_load(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void look_store(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// KI: type of the keys read (int64_t codes in the first pass), KO: type of the keys kept between passes.
// totals: this pass's digit totals of every row [k][256]; look: the tiles' published counts [k][tiles][256].
template <typename KI, typename KO, bool FIRST, bool LAST>
__global__ __launch_bounds__(SORT_THREADS) void scatter_kernel(
    const KI* __restrict__ keys_in, const int32_t* __restrict__ idx_in, int64_t n, int shift, int pass,
    const uint32_t* __restrict__ totals, uint64_t* look, int tiles, uint32_t* __restrict__ gave_up,
    KO* __restrict__ keys_out, int32_t* __restrict__ idx_out, int64_t* __restrict__ order,
    int64_t* __restrict__ inverse) {
    __shared__ uint32_t whist[SORT_WAVES][RADIX];   // per wave and digit: count, then start inside the sorted tile
    __shared__ uint32_t gdelta[RADIX];              // global start of the digit's run minus its start inside the tile
    __shared__ uint32_t wsum[SORT_WAVES];
    __shared__ uint32_t dbase[RADIX];               // inclusive scan of the row's digit totals
    extern __shared__ __align__(16) unsigned char sort_smem[];   // the tile in digit order: keys, then indices
    KO* skey = (KO*)sort_smem;
    int32_t* sidx = (int32_t*)(sort_smem + sizeof(KO) * SORT_TILE);
    const int row = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / PTV3_WAVE, lane = tid % PTV3_WAVE;
    for (int e = tid; e < SORT_WAVES * RADIX; e += SORT_THREADS) (&whist[0][0])[e] = 0;
    const uint32_t total_d = tid < RADIX ? totals[row * RADIX + tid] : 0u;   // keys of digit `tid` in the whole row
    if (tid < RADIX) dbase[tid] = total_d;
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
    __syncthreads();
    // digit `tid` (the first 256 threads = four whole waves): publish the tile's count, then its start inside the
    // sorted tile (exclusive scan of the tile histogram over the digits) and the starts of each wave's run of it
    const uint32_t s_counts = 2u * (uint32_t)pass + 1u, s_sums = s_counts + 1u;
    uint64_t* my_word = look + ((int64_t)row * tiles + tile) * RADIX + tid;
    uint32_t c[SORT_WAVES], total = 0, x = 0;
    if (tid < RADIX) {
#pragma unroll
        for (int w = 0; w < SORT_WAVES; ++w) { c[w] = whist[w][tid]; total += c[w]; }
        look_store(my_word, ((uint64_t)(tile == 0 ? s_sums : s_counts) << 32) | total);
        x = total;
#pragma unroll
        for (int off = 1; off < PTV3_WAVE; off <<= 1) {
            const uint32_t y = __shfl_up(x, off, PTV3_WAVE);
            if (lane >= off) x += y;
        }
        if (lane == PTV3_WAVE - 1) wsum[wave] = x;
    }
    // inclusive scan of the row's digit totals over the 256 digits
    for (int off = 1; off < RADIX; off <<= 1) {
        const uint32_t v = (tid < RADIX && tid >= off) ? dbase[tid - off] : 0u;
        __syncthreads();
        if (tid < RADIX) dbase[tid] += v;
        __syncthreads();
    }
    if (tid < RADIX) {
        // keys of this digit in the tiles in front: walk back over their words, sixteen at a time (one round trip),
        // up to the first inclusive sum
        uint32_t before = 0;
        bool timed_out = false;
        for (int t = tile - 1; t >= 0;) {
            constexpr int CH = 16;
            uint64_t w[CH];
            const uint64_t* p = look + ((int64_t)row * tiles + t) * RADIX + tid;
#pragma unroll
            for (int j = 0; j < CH; ++j) w[j] = t - j >= 0 ? look_load(p - (int64_t)j * RADIX) : 0ull;
            bool closed = false;
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                if (closed || t - j < 0) continue;
                for (int spin = 0; (uint32_t)(w[j] >> 32) < s_counts; ++spin) {
                    if (spin >= SPIN_LIMIT) { timed_out = true; break; }
                    __builtin_amdgcn_s_sleep(1);
                    w[j] = look_load(p - (int64_t)j * RADIX);
                }
                before += (uint32_t)w[j];
                closed = (uint32_t)(w[j] >> 32) >= s_sums;
            }
            if (closed || timed_out) break;
            t -= CH;
        }
        if (timed_out) atomicOr(gave_up, 1u);
        if (tile > 0) look_store(my_word, ((uint64_t)s_sums << 32) | (before + total));
        uint32_t start = x - total;
        for (int w = 0; w < wave; ++w) start += wsum[w];
        gdelta[tid] = dbase[tid] - total_d + before - start;
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
    uint32_t* totals;   // [MAX_PASSES][k][RADIX], then one word: a look-back gave up waiting
    uint64_t* look;     // [k][tiles][RADIX]
    size_t zero_words;  // 32-bit words from `totals` on that are cleared before a sort
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
    const size_t zero_from = off;
    w.totals = (uint32_t*)(p + off);
    off += ptv3_align256(((size_t)MAX_PASSES * k * RADIX + 1) * sizeof(uint32_t));
    w.look = (uint64_t*)(p + off);
    off += ptv3_align256((size_t)k * tiles * RADIX * sizeof(uint64_t));
    w.zero_words = (off - zero_from) / sizeof(uint32_t);
    w.bytes = off;
    return w;
}

template <typename KO>
int run_passes(const int64_t* code, int64_t n, int k, int passes, int64_t* order, int64_t* inverse, const SortWs& w,
                hipStream_t stream) {
    const int tiles = (int)ptv3_ceil_div(n, SORT_TILE);
    const size_t lds = (sizeof(KO) + sizeof(int32_t)) * SORT_TILE;
    const dim3 grid((unsigned)tiles, (unsigned)k), block(SORT_THREADS);
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)ptv3_ceil_div((int64_t)w.zero_words, 256)), dim3(256), 0, stream,
                       w.totals, (int64_t)w.zero_words);
    hipLaunchKernelGGL(digit_totals_kernel, grid, block, 0, stream, code, n, passes, k, w.totals);
    uint32_t* gave_up = w.totals + (size_t)MAX_PASSES * k * RADIX;
    const KO* kin = nullptr;
    const int32_t* iin = nullptr;
    for (int p = 0; p < passes; ++p) {
        const int shift = 8 * p;
        const bool first = (p == 0), last = (p == passes - 1);
        KO* kout = (KO*)w.keys[p & 1];
        int32_t* iout = w.idx[p & 1];
        const uint32_t* totals = w.totals + (size_t)p * k * RADIX;
#define PTV3_SCATTER(KI, IN, F, L)                                                                          \
    do {                                                                                                    \
        auto kern = scatter_kernel<KI, KO, F, L>;                                                           \
        static LdsGrant grant; /* per instantiation and device: the tile needs more than the default 64 KB */ \
        if (const int rc_ = ptv3_allow_lds((const void*)kern, lds, grant)) return rc_;                      \
        hipLaunchKernelGGL(kern, grid, block, lds, stream, IN, iin, n, shift, p, totals, w.look, tiles, gave_up, kout, \
                           iout, order, inverse);                                                           \
    } while (0)
        if (first && last) PTV3_SCATTER(int64_t, code, true, true);
        else if (first) PTV3_SCATTER(int64_t, code, true, false);
        else if (last) PTV3_SCATTER(KO, kin, false, true);
        else PTV3_SCATTER(KO, kin, false, false);
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
