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

// The tasks of a 64-row list sorted into two index lists by their number of rows: out[0] = tasks of at most 32 rows, out[1] =
// tasks of 33..64 rows, out[2 .. 2 + bound) the first kind's task indices in list order, out[2 + bound .. 2 + 2 bound) the
// second kind's. Of an expert's tasks only the last can have fewer than 64 rows, so the lists follow from the counts alone:
// the same block of 512 threads that wrote the task list writes them, from three more scans (experts <= 512).
__device__ __forceinline__ void task_class_lists_block(const uint32_t* __restrict__ counts, uint32_t* __restrict__ out, uint32_t experts,
                                                       uint32_t selected, uint32_t tokens, bool every_token, uint32_t* scan_all,
                                                       uint32_t* scan_small, uint32_t* scan_large) {
    constexpr uint32_t tile = 64;
    const uint32_t tid = threadIdx.x;
    const uint32_t extra = every_token ? (tokens + tile - 1) / tile : 0;
    const uint32_t bound = tokens * selected / tile + experts + extra;
    const uint32_t count = tid < experts ? (counts[tid] < tokens ? counts[tid] : tokens) : 0;
    const uint32_t n = (count + tile - 1) / tile;
    const uint32_t small = n && count - (n - 1) * tile <= 32 ? 1 : 0;  // the last task is a small one
    __syncthreads();
    scan_all[tid] = n;
    scan_small[tid] = small;
    scan_large[tid] = n - small;
    __syncthreads();
    for (uint32_t step = 1; step < 512; step <<= 1) {
        const uint32_t a = tid >= step ? scan_all[tid - step] : 0, b = tid >= step ? scan_small[tid - step] : 0, c = tid >= step ? scan_large[tid - step] : 0;
        __syncthreads();
        scan_all[tid] += a;
        scan_small[tid] += b;
        scan_large[tid] += c;
        __syncthreads();
    }
    const uint32_t total = scan_all[511], total_small = scan_small[511], total_large = scan_large[511];
    const uint32_t first = scan_all[tid] - n, first_small = scan_small[tid] - small, first_large = scan_large[tid] - (n - small);
    uint32_t* list_small = out + 2;
    uint32_t* list_large = out + 2 + bound;
    for (uint32_t i = 0; i < n; ++i) {
        if (first + i >= bound) break;
        if (small && i + 1 == n) list_small[first_small] = first + i;
        else list_large[first_large + i] = first + i;
    }
    const uint32_t extra_small = extra && tokens - (extra - 1) * tile <= 32 ? 1 : 0;
    for (uint32_t i = tid; i < extra; i += 512) {
        if (total + i >= bound) break;
        if (extra_small && i + 1 == extra) list_small[total_small] = total + i;
        else list_large[total_large + i] = total + i;
    }
    if (tid == 0) {
        const bool fits = total + extra <= bound;  // otherwise the task list itself is flagged as broken and nobody reads these
        out[0] = fits ? total_small + extra_small : 0;
        out[1] = fits ? total_large + extra - extra_small : 0;
    }
}

}  // namespace tsp
