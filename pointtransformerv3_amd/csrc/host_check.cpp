// Host build of the per-point code arithmetic, for CPU-side checks of the kernel math.
// Not part of libptv3_hip.so.
#include "encode_core.h"

extern "C" void ptv3_host_curve_codes(const int32_t* grid_coord, int64_t n, int depth, int id,
                                      int64_t* out) {
    const uint32_t mask = (1u << depth) - 1u;
    for (int64_t p = 0; p < n; ++p)
        out[p] = (int64_t)ptv3::curve_code(id, (uint32_t)grid_coord[3 * p] & mask,
                                           (uint32_t)grid_coord[3 * p + 1] & mask,
                                           (uint32_t)grid_coord[3 * p + 2] & mask, depth);
}
