// Deterministic expert permutation, prefix-sum tile offsets, and the T <= 8 union records.
// Integer work only; every output word is a pure function of the route ids, so results are
// bit-identical run to run and identical to the sequential specification.
//
//  grouped_routes  token_map[e*T + k] = t*S + slot for the k-th token (ascending) that routes to e;
//                  counts[e] = number of such tokens. No atomics on the map: one block per expert
//                  compacts with ballots and a running base, so order is the token order.
//  grouped_tasks   tiles(e) = ceil(min(counts[e], T) / tile); exclusive scan over experts; task i of
//                  expert e is (e, i*tile); unused slots up to the bound are 0xFFFFFFFF.
//  union_build     for T*S <= 128 routes: records (expert, <= cap routes) in first-use order.
#include "grouping_device.hpp"

using namespace tsp;

namespace {

constexpr uint32_t kRouteThreads = 1024;  // tokens looked at per pass of one expert's workgroup

__global__ __launch_bounds__(kRouteThreads) void grouped_routes_kernel(const uint32_t* __restrict__ ids, uint32_t* __restrict__ token_map,
                                                             uint32_t* __restrict__ counts, uint32_t experts, uint32_t selected,
                                                             uint32_t tokens, uint32_t* error_word) {
    __shared__ uint32_t wave_totals[kRouteThreads / kWave];
    const uint32_t expert = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    uint32_t accumulated = 0, bad = 0;
    for (uint32_t base = 0; base < tokens; base += kRouteThreads) {
        const uint32_t token = base + tid;
        uint32_t slot = 0xffffffffu, matches = 0;
        if (token < tokens) {
            const uint32_t* row = ids + uint64_t(token) * selected;
            if (selected % 2 == 0 && reinterpret_cast<uintptr_t>(ids) % 8 == 0) {  // 8-byte aligned rows of an even number of ids: half as many loads
                for (uint32_t i = 0; i < selected; i += 2) {
                    const uint2 pair = *reinterpret_cast<const uint2*>(row + i);
                    if (pair.x >= experts || pair.y >= experts) bad = TSP_ERRBIT_INDEX;
                    if (pair.x == expert) { slot = i; ++matches; }
                    if (pair.y == expert) { slot = i + 1; ++matches; }
                }
            } else {
                for (uint32_t i = 0; i < selected; ++i) {
                    const uint32_t id = row[i];
                    if (id >= experts) bad = TSP_ERRBIT_INDEX;
                    if (id == expert) { slot = i; ++matches; }
                }
            }
        }
        if (matches > 1) bad = TSP_ERRBIT_INDEX;
        const bool found = matches == 1;
        const uint64_t mask = __builtin_amdgcn_ballot_w64(found);
        const uint32_t prefix = __builtin_popcountll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_totals[wave] = __builtin_popcountll(mask);
        __syncthreads();
        uint32_t before = 0, chunk = 0;
        for (uint32_t w = 0; w < kRouteThreads / kWave; ++w) { if (w < wave) before += wave_totals[w]; chunk += wave_totals[w]; }
        if (found) token_map[uint64_t(expert) * tokens + accumulated + before + prefix] = token * selected + slot;
        accumulated += chunk;
        __syncthreads();
    }
    if (tid == 0) counts[expert] = accumulated;
    publish_error(bad, error_word);
}

// Block b writes list b: the same counts tiled two ways in one launch (tasks1 may be null with a grid of one).
__global__ __launch_bounds__(512) void grouped_tasks_kernel(const uint32_t* __restrict__ counts, uint32_t* __restrict__ tasks0, uint32_t tile0,
                                                            uint32_t* __restrict__ tasks1, uint32_t tile1, uint32_t experts, uint32_t selected,
                                                            uint32_t tokens, uint32_t* error_word) {
    __shared__ uint32_t tiles_scan[512];
    __shared__ uint32_t routes_scan[512];
    grouped_tasks_block(counts, blockIdx.x == 0 ? tasks0 : tasks1, blockIdx.x == 0 ? tile0 : tile1, experts, selected, tokens, error_word,
                        tiles_scan, routes_scan);
}

// 128 threads, one per flat route (T*S <= 128); the block's layout and arithmetic: union_block (grouping_device.hpp).
__global__ __launch_bounds__(128) void union_build_kernel(const uint32_t* __restrict__ ids, uint32_t* __restrict__ meta,
                                                          uint32_t experts, uint32_t selected, uint32_t tokens, uint32_t hidden,
                                                          uint32_t channels, uint32_t* error_word) {
    __shared__ __align__(16) uint32_t scratch[kUnionScratchWords];
    const uint32_t f = threadIdx.x;
    // the shape test comes again inside; here it only keeps the read of ids in bounds
    const bool readable = tokens && tokens <= 8 && selected && selected <= 16 && f < tokens * selected;
    const uint32_t mine = readable ? ids[f] : 0xffffffffu;
    union_block(mine, f, 128u, experts, selected, tokens, hidden, channels, scratch,
                [&](uint32_t word, uint32_t value) { meta[word] = value; }, [&]() { atomicOr(error_word, TSP_ERRBIT_INDEX); });
}

}  // namespace

extern "C" int tsp_grouped_routes(const uint32_t* ids, uint32_t* token_map, uint32_t* counts, uint32_t experts, uint32_t selected,
                                  uint32_t tokens, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(experts && experts <= 512 && selected && selected <= 16 && selected <= experts && tokens && tokens <= 2048,
                "grouped routes geometry");
    TSP_REQUIRE(ids && token_map && counts && error_word, "null device pointer");
    TSP_LAUNCH("grouped_routes", static_cast<hipStream_t>(stream), grouped_routes_kernel<<<experts, kRouteThreads, 0, static_cast<hipStream_t>(stream)>>>(ids, token_map, counts, experts, selected, tokens, error_word));
    return launch_status("grouped_routes");
}

extern "C" int tsp_grouped_tasks(const uint32_t* counts, uint32_t* tasks, uint32_t experts, uint32_t selected, uint32_t tokens,
                                 uint32_t tile, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(experts && experts <= 512 && selected && selected <= 16 && tokens && tokens <= 2048 && tile && tile <= 256,
                "grouped tasks geometry");
    TSP_REQUIRE(counts && tasks && error_word, "null device pointer");
    TSP_LAUNCH("grouped_tasks", static_cast<hipStream_t>(stream), grouped_tasks_kernel<<<1, 512, 0, static_cast<hipStream_t>(stream)>>>(counts, tasks, tile, nullptr, 0, experts, selected, tokens, error_word));
    return launch_status("grouped_tasks");
}

extern "C" int tsp_planar_union_build(const uint32_t* ids, uint32_t* meta, uint32_t experts, uint32_t selected, uint32_t tokens,
                                      uint32_t hidden, uint32_t channels, uint32_t* error_word, void* stream) {
    // Shape validity is decided on the device like the engine's kernel (it flags and zeroes the header);
    // only what would index outside the 128-route staging is refused here.
    TSP_REQUIRE(uint64_t(tokens) * selected <= 128 || !(tokens <= 8 && selected <= 16), "union build route bound");
    TSP_REQUIRE(ids && meta && error_word, "null device pointer");
    TSP_LAUNCH("union_build", static_cast<hipStream_t>(stream), union_build_kernel<<<1, 128, 0, static_cast<hipStream_t>(stream)>>>(ids, meta, experts, selected, tokens, hidden, channels, error_word));
    return launch_status("planar_union_build");
}
