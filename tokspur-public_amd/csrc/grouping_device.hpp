// Device code shared by grouping.hip, gemm.hip and record_resident.hip: the task list of the grouped GEMMs and the union
// records of a step of at most eight tokens.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

// Inclusive sums over the 512 values of a block of 512 threads (one per thread), two or three sequences at once: each wave
// scans its 64 values with six shuffles, the eight wave totals meet in LDS (`totals`: 8 words per sequence), one barrier on
// the way in and one on the way out, where a step-by-step scan through LDS takes eighteen. Returns the scan at this thread;
// `grand[i]` receives the sum of all 512.
template <int N>
__device__ __forceinline__ void scan512(uint32_t (&v)[N], uint32_t (&grand)[N], uint32_t* totals) {
    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
#pragma unroll
    for (int i = 0; i < N; ++i) {
#pragma unroll
        for (int step = 1; step < kWave; step <<= 1) {
            const uint32_t below = uint32_t(__shfl_up(int(v[i]), step, kWave));
            if (lane >= uint32_t(step)) v[i] += below;
        }
    }
    __syncthreads();  // whoever still reads `totals` from an earlier call has left
    if (lane == kWave - 1)
#pragma unroll
        for (int i = 0; i < N; ++i) totals[i * 8 + wave] = v[i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        uint32_t before = 0, all = 0;
#pragma unroll
        for (uint32_t w = 0; w < 8; ++w) { const uint32_t t = totals[i * 8 + w]; if (w < wave) before += t; all += t; }
        v[i] += before;
        grand[i] = all;
    }
}

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
    uint32_t scans[2] = {n, count}, sums[2];
    scan512(scans, sums, tiles_scan);
    (void)routes_scan;
    const uint32_t total = sums[0], routes = sums[1];
    const uint32_t offset = scans[0] - n;
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
    uint32_t scans[3] = {n, small, n - small}, sums[3];
    scan512(scans, sums, scan_all);
    (void)scan_small; (void)scan_large;
    const uint32_t total = sums[0], total_small = sums[1], total_large = sums[2];
    const uint32_t first = scans[0] - n, first_small = scans[1] - small, first_large = scans[2] - (n - small);
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

// The union records of at most 128 routes (T <= 8 tokens x S <= 16 slots): records (expert, <= cap routes) in first-use
// order. Block layout in 32-bit words: [0..7] header, +8 experts[128], +136 counts[128], +264 tokens[128][8],
// +1288 routes[128][8]. Thread f < 128 owns flat route f and brings its expert id (`mine`, anything when f >= T S); threads
// from 128 on help clear the scratch and keep the barriers company. `scratch`: kUnionScratchWords of LDS, 16-byte aligned.
// `store(word, value)` puts a word of the block wherever the caller wants it. Returns false, with the header zeroed and
// `raise()` called by thread 0, when the shape or an id is out of range. Uniform over the workgroup; every thread must call.
//
// A route's rank among the routes of its expert is a population count: every expert has a 128-bit set of its routes (bit f:
// route f), filled by LDS atomics whose result does not depend on their order, and route f counts the bits below its own. The
// route that opened a record is found the same way, as the n-th set bit of the expert's set, so nothing scans the routes.
constexpr uint32_t kUnionScratchWords = 512 * 4 + 128 + 4;
__device__ __forceinline__ uint32_t nth_set_bit(uint32_t word, uint32_t n) {  // position of the (n + 1)-th set bit; it must exist
    uint32_t pos = 0;
#pragma unroll
    for (uint32_t half = 16; half >= 1; half >>= 1) {
        const uint32_t low = word & ((1u << half) - 1u), in_low = __builtin_popcount(low);
        if (n < in_low) { word = low; } else { n -= in_low; word >>= half; pos += half; }
    }
    return pos;
}
template <typename Store, typename Raise>
__device__ __forceinline__ bool union_block(uint32_t mine, uint32_t f, uint32_t threads, uint32_t experts, uint32_t selected, uint32_t tokens,
                                            uint32_t hidden, uint32_t channels, uint32_t* scratch, Store store, Raise raise) {
    uint32_t* const sets = scratch;                  // [512][4]
    uint32_t* const record_of = scratch + 2048;      // [128]: the record a route opened
    uint32_t* const wave_leaders = scratch + 2176;   // [2]
    uint32_t* const any_bad = scratch + 2178;
    const uint32_t total = tokens * selected;
    const bool shape_ok = experts && experts <= 512 && experts % 2 == 0 && selected && selected <= 16 && selected <= experts &&
                          tokens && tokens <= 8 && hidden && channels;
    for (uint32_t i = f; i < 2048; i += threads) sets[i] = 0;
    if (f == 0) *any_bad = shape_ok ? 0u : 1u;
    __syncthreads();
    const bool live = shape_ok && f < total;
    if (live) {
        if (mine >= experts) *any_bad = 1u;
        else atomicOr(&sets[mine * 4 + f / 32], 1u << (f % 32));
    }
    __syncthreads();
    if (*any_bad) {
        if (f < 8) store(f, 0u);
        if (f == 0) raise();
        return false;
    }
    const uint32_t cap = tokens <= 4 ? 4u : 8u;
    uint32_t set[4] = {0, 0, 0, 0}, rank = 0, same = 0;
    if (live) {
        const uint4 four = *reinterpret_cast<const uint4*>(&sets[mine * 4]);
        set[0] = four.x; set[1] = four.y; set[2] = four.z; set[3] = four.w;
#pragma unroll
        for (uint32_t w = 0; w < 4; ++w) {
            same += __builtin_popcount(set[w]);
            const uint32_t below = w < f / 32 ? set[w] : w == f / 32 ? set[w] & ((1u << (f % 32)) - 1u) : 0u;
            rank += __builtin_popcount(below);
        }
    }
    const bool leader = live && rank % cap == 0;
    const uint64_t mask = __builtin_amdgcn_ballot_w64(leader);
    const uint32_t lane = f % kWave, wave = f / kWave;
    if (lane == 0 && wave < 2) wave_leaders[wave] = __builtin_popcountll(mask);
    __syncthreads();
    const uint32_t record = (wave ? wave_leaders[0] : 0u) + __builtin_popcountll(mask & ((1ull << lane) - 1ull));
    const uint32_t records = wave_leaders[0] + wave_leaders[1];
    if (leader) record_of[f] = record;
    __syncthreads();
    if (live) {
        uint32_t rec = record;
        if (!leader) {
            // my record is the one opened by the route of my expert whose rank is rank - rank % cap
            uint32_t n = rank - rank % cap, opener = 0;
            bool found = false;
#pragma unroll
            for (uint32_t w = 0; w < 4; ++w) {
                const uint32_t here = __builtin_popcount(set[w]);
                if (!found && n < here) { opener = 32 * w + nth_set_bit(set[w], n); found = true; }
                if (!found) n -= here;
            }
            rec = record_of[opener];
        }
        const uint32_t slot = rank % cap;
        store(264 + rec * 8 + slot, f / selected);
        store(1288 + rec * 8 + slot, f);
        if (leader) {
            const uint32_t members = same - rank < cap ? same - rank : cap;
            store(8 + rec, mine);
            store(136 + rec, members);
            for (uint32_t k = members; k < 8; ++k) { store(264 + rec * 8 + k, f / selected); store(1288 + rec * 8 + k, f); }
        }
    }
    if (f == 0) {
        store(0, (hidden + 7) / 8); store(1, records); store(2, 1u);
        store(3, (channels + 15) / 16); store(4, records); store(5, 1u);
        store(6, records); store(7, 0u);
    }
    return true;
}

}  // namespace tsp
