// A plain device-to-device copy of a known size. Hardware counter readings for a kernel (bytes fetched from and
// written to HBM) are scaled by what the same counters read for this copy, whose traffic is known exactly.
#include "tsp_common.hpp"

using namespace tsp;

namespace {
__global__ __launch_bounds__(256) void calibration_copy(const uint4* __restrict__ src, uint4* __restrict__ dst, uint64_t chunks) {
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < chunks; i += uint64_t(gridDim.x) * blockDim.x) dst[i] = src[i];
}
}  // namespace

extern "C" int tsp_calibration_copy(void* dst, const void* src, uint64_t bytes, void* stream) {
    TSP_REQUIRE(dst && src && bytes && bytes % 16 == 0, "calibration copy takes a non-empty multiple of 16 bytes");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(dst) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0, "calibration copy needs 16-byte alignment");
    TSP_REQUIRE(!ranges_overlap(dst, bytes, src, bytes), "calibration copy buffers overlap");
    const uint64_t chunks = bytes / 16;
    const uint32_t grid = uint32_t((chunks + 255) / 256 > 16384 ? 16384 : (chunks + 255) / 256);
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("calibration_copy", s, calibration_copy<<<grid, 256, 0, s>>>(static_cast<const uint4*>(src), static_cast<uint4*>(dst), chunks));
    return launch_status("calibration_copy");
}
