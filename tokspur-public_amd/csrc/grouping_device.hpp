// Device code shared by grouping.hip and gemm.hip: the task list of the grouped GEMMs.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

// One block of 512 threads writes one list; experts <= 512. tiles(e) = ceil(min(counts[e], T) / tile), exclusive scan over
// the experts, task i of expert e is (e, i * tile); unused slots up to the bound are 0xFFFFFFFF. The two scan arrays (512
// words each) are the caller's LDS.
// `every_token` appends ceil(tokens / tile) tasks (experts, i * tile) after the experts' own: an always-on expert whose rows
// are the tokens themselves (the bound grows by that many slots).
__device__ __forceinline__ void grouped_tasks_block(const uint32_t* __restrict__ counts, uint32_t* __restrict__ tasks, uint32_t tile,
                                                    uint32_t experts, uint32_t selected, uint32_t tokens, uint32_t* error_word,
                                                    uint32_t* tiles_scan, uint32_t* routes_scan, bool every_token = false) {
    const uint32_t tid = threadIdx.x;
    const uint32_t extra = every_token ? (tokens + tile - 1) / tile : 0;
    const uint32_t bound = tokens * selected / tile + experts + extra;
    uint32_t bad = 0;
    const uint32_t count = tid < experts ? counts[tid] : 0;
    if (count > tokens) bad = TSP_ERRBIT_INDEX;
    const uint32_t n = ((count < tokens ? count : tokens) + tile - 1) / tile;
    tiles_scan[tid] = n;
    routes_scan[tid] = count;
    __syncthreads();
    for (uint32_t step = 1; step < 512; step <<= 1) {  // inclusive Hillis-Steele scan
        const uint32_t a = tid >= step ? tiles_scan[tid - step] : 0, b = tid >= step ? routes_scan[tid - step] : 0;
        __syncthreads();
        tiles_scan[tid] += a;
        routes_scan[tid] += b;
        __syncthreads();
    }
    const uint32_t total = tiles_scan[511], routes = routes_scan[511];
    const uint32_t offset = tiles_scan[tid] - n;
    for (uint32_t i = tid; i < bound; i += 512) { tasks[2 + 2 * i] = 0xffffffffu; tasks[3 + 2 * i] = 0xffffffffu; }
    __syncthreads();
    if (tid < experts)
        for (uint32_t i = 0; i < n; ++i)
            if (offset + i < bound) { tasks[2 + 2 * (offset + i)] = tid; tasks[3 + 2 * (offset + i)] = i * tile; }
    for (uint32_t i = tid; i < extra; i += 512)
        if (total + i < bound) { tasks[2 + 2 * (total + i)] = experts; tasks[3 + 2 * (total + i)] = i * tile; }
    if (tid == 0) {
        tasks[0] = total + extra < bound ? total + extra : bound;
        tasks[1] = routes;
        if (total + extra > bound || routes != tokens * selected) bad = TSP_ERRBIT_INDEX;
    }
    publish_error(bad, error_word);
}

}  // namespace tsp
