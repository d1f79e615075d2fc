// Space-filling-curve codes for all requested orders in one pass over the points, and their inverse.
//
// Replaces serialization/default.py:8-24 with z_order.py:66-101 and hilbert.py:91-198 of the
// reference: one thread per point, coordinates stay in registers, the k codes are written
// as k coalesced int64 streams. HBM traffic is the algorithmic minimum
// (12 B coords + 8 B batch in, 8*k B out per point).
#include "common.h"
#include "encode_core.h"

namespace {

struct OrderList { int id[8]; };

__global__ __launch_bounds__(256) void encode_kernel(const int32_t* __restrict__ grid_coord,
                                                     const int64_t* __restrict__ batch,
                                                     int64_t n, int depth, OrderList orders, int k,
                                                     int64_t* __restrict__ code) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n) return;
    const uint32_t mask = (1u << depth) - 1u;   // depth <= 16
    const uint32_t x = (uint32_t)grid_coord[3 * p + 0] & mask;
    const uint32_t y = (uint32_t)grid_coord[3 * p + 1] & mask;
    const uint32_t z = (uint32_t)grid_coord[3 * p + 2] & mask;
    const uint64_t hi = batch ? ((uint64_t)batch[p] << (3 * depth)) : 0ull;
    for (int r = 0; r < k; ++r) {
        const int id = orders.id[r];
        const uint64_t c = ptv3::curve_code(id, x, y, z, depth);
        code[(int64_t)r * n + p] = (int64_t)(hi | c);
    }
}

// serialization/default.py:27-39: the batch index is what sits above the 3 depth curve bits
__global__ __launch_bounds__(256) void decode_kernel(const int64_t* __restrict__ code, int64_t n, int depth, int id,
                                                     int64_t* __restrict__ grid_coord, int64_t* __restrict__ batch) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n) return;
    const int64_t c = code[p];
    const uint64_t low = (uint64_t)c & ((1ull << (3 * depth)) - 1ull);   // depth <= 16: at most 48 bits
    uint32_t x, y, z;
    ptv3::curve_point(id, low, depth, x, y, z);
    grid_coord[3 * p + 0] = x;
    grid_coord[3 * p + 1] = y;
    grid_coord[3 * p + 2] = z;
    if (batch) batch[p] = c >> (3 * depth);   // arithmetic shift, as torch's >> on int64
}

}  // namespace

extern "C" int ptv3_decode(const int64_t* code, int64_t n, int depth, int order_id, int64_t* grid_coord,
                           int64_t* batch, void* stream) {
    if (n < 0 || order_id < 0 || order_id > 3) return PTV3_EINVAL;
    if (depth < 1 || depth > 16) return PTV3_EDEPTH;
    if (n == 0) return PTV3_OK;
    if (!code || !grid_coord) return PTV3_EINVAL;
    hipLaunchKernelGGL(decode_kernel, dim3((unsigned)ptv3_ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream,
                       code, n, depth, order_id, grid_coord, batch);
    PTV3_RETURN_LAUNCH();
}

extern "C" int ptv3_encode(const int32_t* grid_coord, const int64_t* batch, int64_t n, int depth,
                           const int32_t* order_ids_host, int k, int64_t* code, void* stream) {
    if (n < 0 || k < 1 || k > 8 || !order_ids_host) return PTV3_EINVAL;
    if (depth < 1 || depth > 16) return PTV3_EDEPTH;
    OrderList ol;
    for (int r = 0; r < 8; ++r) ol.id[r] = 0;
    for (int r = 0; r < k; ++r) {
        if (order_ids_host[r] < 0 || order_ids_host[r] > 3) return PTV3_EINVAL;
        ol.id[r] = order_ids_host[r];
    }
    if (n == 0) return PTV3_OK;
    if (!grid_coord || !code) return PTV3_EINVAL;
    const int threads = 256;
    const int64_t blocks = ptv3_ceil_div(n, threads);
    hipLaunchKernelGGL(encode_kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream,
                       grid_coord, batch, n, depth, ol, k, code);
    PTV3_RETURN_LAUNCH();
}
