// Microbenchmarks of the part itself (not of this package's kernels): instruction issue rates and vector-load
// throughput by access pattern. The figures the kernel designs lean on come from here: a v_exp_f32 occupies the
// VALU issue port for 8 cycles (so the softmax, not the MFMAs, bounds attention at head_dim 16); a load instruction
// that touches 32 rows of 32 bytes runs at the texture path's line rate, far below one contiguous KB per
// instruction (so operands are gathered in whole row segments and converted through LDS).
// Built into libptv3_micro.so, beside the product library; `bench.py --micro issue|loads` prints the report.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <string>

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define MICRO_CHECK(x)                                                      \
    do {                                                                    \
        hipError_t e__ = (x);                                               \
        if (e__ != hipSuccess) return (int)e__;                             \
    } while (0)

// ---- issue rates: one wave per SIMD (or four) issues the same instruction back to back, 8 independent chains.
// Times are per instruction and SIMD, and as multiples of v_max_f32's under the same number of waves (the clock the
// part sustains depends on what the loop does, so nanoseconds of different loops do not convert at one clock).
template <int OP>
__global__ __launch_bounds__(256) void issue_kernel(float* out, int iters) {
    float a[8];
    for (int i = 0; i < 8; ++i) a[i] = threadIdx.x * 0.001f + i;
    f32x16 acc = {0};
    f32x4 acc4 = {0};
    f16x8 fa, fb;
    for (int i = 0; i < 8; ++i) { fa[i] = (_Float16)(threadIdx.x & 3); fb[i] = (_Float16)1; }
    uint32_t u[8];
    for (int i = 0; i < 8; ++i) u[i] = threadIdx.x * 77 + i;
    for (int it = 0; it < iters; ++it) {
        if (OP == 0) { for (int i = 0; i < 8; ++i) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(a[i])); }
        if (OP == 1) { for (int i = 0; i < 8; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(a[i])); }
        if (OP == 2) { for (int i = 0; i < 8; ++i) asm volatile("v_exp_f16 %0, %0" : "+v"(a[i])); }
        if (OP == 3) { for (int i = 0; i < 8; ++i) asm volatile("v_pk_fma_f16 %0, %0, %0, %0" : "+v"(a[i])); }
        if (OP == 4) { for (int i = 0; i < 8; ++i) asm volatile("v_rcp_f32 %0, %0" : "+v"(a[i])); }
        if (OP == 5) { for (int i = 0; i < 8; ++i) asm volatile("v_cvt_pkrtz_f16_f32 %0, %0, %0" : "+v"(a[i])); }
        if (OP == 6) { for (int i = 0; i < 8; ++i) asm volatile("v_max_f32 %0, %0, %0" : "+v"(a[i])); }
        if (OP == 7) { for (int i = 0; i < 8; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc, 0, 0, 0); }
        if (OP == 8) { for (int i = 0; i < 8; ++i) acc4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fb, acc4, 0, 0, 0); }
        if (OP == 9) {   // one MFMA and two exponentials per group: does the matrix pipe run under the VALU?
            for (int i = 0; i < 8; ++i) {
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc, 0, 0, 0);
                asm volatile("v_exp_f32 %0, %0" : "+v"(a[i]));
                asm volatile("v_exp_f32 %0, %0" : "+v"(a[(i + 4) & 7]));
            }
        }
        if (OP == 10) {   // one exponential and two FMAs per group: does the transcendental unit run beside the VALU?
            for (int i = 0; i < 4; ++i) {
                asm volatile("v_exp_f32 %0, %0" : "+v"(a[i]));
                asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(a[i + 4]));
                asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(a[i + 4]));
            }
        }
        if (OP == 11) { for (int i = 0; i < 8; ++i) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %0" : "+v"(a[i])); }
    }
    float s = 0;
    for (int i = 0; i < 8; ++i) s += a[i] + u[i];
    for (int i = 0; i < 16; ++i) s += acc[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s + acc4[0];
}

template <int OP>
int issue_case(std::string& rep, const char* name, float* d, int per_iter, int waves_per_simd, double* base_ns) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    MICRO_CHECK(hipEventCreate(&e0));
    MICRO_CHECK(hipEventCreate(&e1));
    const dim3 grid(256 * waves_per_simd), block(256);   // four waves per work-group: one per SIMD
    hipLaunchKernelGGL(issue_kernel<OP>, grid, block, 0, 0, d, 100);
    MICRO_CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(issue_kernel<OP>, grid, block, 0, 0, d, iters);
    MICRO_CHECK(hipEventRecord(e1));
    MICRO_CHECK(hipEventSynchronize(e1));
    float ms = 0;
    MICRO_CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double ns = ms * 1e6 / ((double)iters * per_iter * waves_per_simd);
    if (OP == 6) *base_ns = ns;
    char line[200];
    snprintf(line, sizeof line, "%-36s %d wave(s) per SIMD: %7.3f ns per instruction and SIMD = %5.2f x v_max_f32\n", name,
             waves_per_simd, ns, ns / *base_ns);
    rep += line;
    MICRO_CHECK(hipEventDestroy(e0));
    MICRO_CHECK(hipEventDestroy(e1));
    return 0;
}

int run_issue(std::string& rep) {
    float* d = nullptr;
    MICRO_CHECK(hipMalloc(&d, (size_t)256 * 4 * 256 * sizeof(float)));
    for (int w : {1, 4}) {
        double base = 1.0;
        int rc = 0;
#define MICRO_ISSUE(OP, name, n) if ((rc = issue_case<OP>(rep, name, d, n, w, &base))) { (void)hipFree(d); return rc; }
        // the unit: a plain VALU instruction, one wave64 through a 16-lane SIMD in 4 cycles
        MICRO_ISSUE(6, "v_max_f32", 8)
        char line[160];
        snprintf(line, sizeof line, "   (if that is 4 cycles, the shader clock under this loop is %.2f GHz)\n", 4.0 / base);
        rep += line;
        MICRO_ISSUE(0, "v_fma_f32", 8) MICRO_ISSUE(1, "v_exp_f32", 8) MICRO_ISSUE(2, "v_exp_f16", 8) MICRO_ISSUE(4, "v_rcp_f32", 8)
        MICRO_ISSUE(5, "v_cvt_pkrtz_f16_f32", 8) MICRO_ISSUE(11, "v_cvt_pk_bf16_f32", 8)
        MICRO_ISSUE(3, "v_pk_fma_f16", 8) MICRO_ISSUE(7, "v_mfma_f32_32x32x16_f16", 8) MICRO_ISSUE(8, "v_mfma_f32_16x16x32_f16", 8)
        MICRO_ISSUE(9, "mfma 32x32x16 + 2 v_exp_f32 (group)", 8) MICRO_ISSUE(10, "v_exp_f32 + 2 v_fma_f32 (group)", 4)
#undef MICRO_ISSUE
    }
    MICRO_CHECK(hipFree(d));
    return 0;
}

// ---- loads: ROWS rows per load instruction (64 / ROWS lanes x 16 B each), rows drawn pseudo-randomly from a working
// set of ws bytes; ROWS = 0: one contiguous KB per instruction
template <int ROWS, int UNROLL>
__global__ __launch_bounds__(256) void load_kernel(const unsigned char* __restrict__ src, size_t ws_bytes, int iters,
                                                   uint32_t* out) {
    const int lane = threadIdx.x & 63, wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    u32x4 acc = {0, 0, 0, 0};
    uint32_t state = wave * 2654435761u + 12345u;
    const size_t rows = ws_bytes / 256;
    for (int it = 0; it < iters; ++it) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            size_t off;
            if (ROWS == 0) {
                state = state * 1664525u + 1013904223u;
                off = ((size_t)(state >> 8) % (ws_bytes / 1024)) * 1024 + lane * 16;
            } else {
                constexpr int LPR = ROWS ? 64 / ROWS : 1;   // lanes per row
                const uint32_t h = (state + (lane / LPR) * 2246822519u + it * 3266489917u + u * 668265263u);
                off = ((size_t)((h ^ (h >> 15)) * 2654435761u >> 4) % rows) * 256 + (lane % LPR) * 16 + (u * LPR * 16) % 256;
            }
            v[u] = *(const u32x4*)(src + off);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc += v[u];
        state += acc[0] & 1;
    }
    out[blockIdx.x * blockDim.x + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}

template <int ROWS>
int load_case(std::string& rep, const char* name, const unsigned char* src, size_t ws, int waves_per_cu, uint32_t* out) {
    constexpr int UNROLL = 8;
    const int iters = 2000;
    hipEvent_t e0, e1;
    MICRO_CHECK(hipEventCreate(&e0));
    MICRO_CHECK(hipEventCreate(&e1));
    const dim3 grid(256 * waves_per_cu / 4), block(256);
    hipLaunchKernelGGL((load_kernel<ROWS, UNROLL>), grid, block, 0, 0, src, ws, 50, out);
    MICRO_CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL((load_kernel<ROWS, UNROLL>), grid, block, 0, 0, src, ws, iters, out);
    MICRO_CHECK(hipEventRecord(e1));
    MICRO_CHECK(hipEventSynchronize(e1));
    float ms = 0;
    MICRO_CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double bytes = (double)grid.x * 4 * iters * UNROLL * 1024.0;
    char line[200];
    snprintf(line, sizeof line, "%-22s working set %7.0f KB, %2d waves per CU: %6.2f TB/s over the chip = %6.1f GB/s per CU\n", name,
             ws / 1024.0, waves_per_cu, bytes / ms / 1e9, bytes / ms / 1e6 / 256);
    rep += line;
    MICRO_CHECK(hipEventDestroy(e0));
    MICRO_CHECK(hipEventDestroy(e1));
    return 0;
}

int run_loads(std::string& rep) {
    const size_t cap = (size_t)512 << 20;
    unsigned char* src = nullptr;
    uint32_t* out = nullptr;
    MICRO_CHECK(hipMalloc(&src, cap));
    MICRO_CHECK(hipMemset(src, 1, cap));
    MICRO_CHECK(hipMalloc(&out, (size_t)256 * 64 * 256 * 4));
    rep += "16-byte loads, 1 KB per wave instruction; rows of 256 B drawn at random from the working set\n";
    for (size_t ws : {(size_t)16 << 10, (size_t)1 << 20, (size_t)24 << 20, (size_t)400 << 20})
        for (int w : {4, 8, 16}) {
            int rc;
            if ((rc = load_case<0>(rep, "1 x 1 KB contiguous", src, ws, w, out))) return rc;
            if ((rc = load_case<4>(rep, "4 rows x 256 B", src, ws, w, out))) return rc;
            if ((rc = load_case<8>(rep, "8 rows x 128 B", src, ws, w, out))) return rc;
            if ((rc = load_case<16>(rep, "16 rows x 64 B", src, ws, w, out))) return rc;
            if ((rc = load_case<32>(rep, "32 rows x 32 B", src, ws, w, out))) return rc;
            if ((rc = load_case<64>(rep, "64 rows x 16 B", src, ws, w, out))) return rc;
        }
    MICRO_CHECK(hipFree(src));
    MICRO_CHECK(hipFree(out));
    return 0;
}

}  // namespace

// which: "issue" or "loads". The report (text) is copied into out (cap bytes, always terminated).
// Returns 0, -1 for an unknown name, or a hipError_t.
extern "C" int ptv3_micro_run(const char* which, char* out, size_t cap) {
    if (!which || !out || cap == 0) return -1;
    std::string rep;
    int rc = -1;
    const std::string w(which);
    if (w == "issue") rc = run_issue(rep);
    else if (w == "loads") rc = run_loads(rep);
    snprintf(out, cap, "%s", rep.c_str());
    return rc;
}
