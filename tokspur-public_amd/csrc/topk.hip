// Row top-64 of a logits matrix: for every row the 64 largest finite logits in the order
// (value descending, column ascending, -0 == +0), the number found, and the first non-finite and first
// subnormal column. Rank 0 is the arg-max a greedy sampler needs.
//
// Two launches. Stage 1: one workgroup per (4096-column tile, row); each of its sixteen waves keeps the 64 largest keys
// of its 256 columns in registers, one key per lane, and the sixteen lists are merged pairwise (a tree through LDS) into
// a partial row. Stage 2: one workgroup per row merges the partial rows' lists the same way and writes the final row. A
// sort or merge is a chain of dependent cross-lane exchanges, so what shortens it is more waves with shorter chains. Keys are 64 bits: high word
// = the float mapped to an unsigned integer of the same order (after -0 -> +0), low word = ~column, so that "largest
// key first" is exactly the ordering above and no two keys are equal. Non-finite logits and padding get key 0, below
// every finite value's key. A list is sorted with a bitonic network over the wave's lanes; two lists are merged by
// sorting one of them ascending, taking the lane-wise maximum (the 64 largest of both, a bitonic sequence) and
// running the last six steps of the network.
#include "tsp_common.hpp"

using namespace tsp;

namespace {

constexpr uint32_t kCapacity = 64, kTileSpan = 4096, kMaxTiles = 256, kNone = 0xffffffffu;
constexpr uint32_t kWaves = 16, kThreads = kWaves * kWave, kWaveSpan = kTileSpan / kWaves;  // 256 columns per wave of stage 1

struct TopKArgs {
    const float* logits;
    uint64_t stride_bytes;
    uint32_t rows, vocabulary, tiles;
    tsp_logit_topk_row* partial;  // [rows][tiles]
    tsp_logit_topk_row* out;      // [rows]
};

__device__ __forceinline__ uint64_t make_key(float value, uint32_t column) {
    uint32_t bits = __float_as_uint(value);
    if ((bits & 0x7f800000u) == 0x7f800000u) return 0;  // inf / nan never rank
    if ((bits & 0x7fffffffu) == 0) bits = 0;             // -0 ranks as +0
    const uint32_t ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return (uint64_t(ordered) << 32) | uint32_t(~column);
}

template <int CTRL>
__device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
    const uint32_t lo = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(v)), CTRL, 0xf, 0xf, true));
    const uint32_t hi = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(v >> 32)), CTRL, 0xf, 0xf, true));
    return (uint64_t(hi) << 32) | lo;
}

// The key of lane (lane ^ STRIDE). Strides 1, 2, 4 and 8 stay inside a row of 16 lanes and use the data-parallel
// primitives (quad permutes, row rotations), whose latency is a fraction of a trip through the LDS crossbar; a sort is
// a chain of 21 dependent exchanges, 18 of them with these strides.
template <uint32_t STRIDE>
__device__ __forceinline__ uint64_t partner(uint64_t key, uint32_t lane) {
    if constexpr (STRIDE == 1) return dpp_u64<0xB1>(key);        // quad_perm [1, 0, 3, 2]
    else if constexpr (STRIDE == 2) return dpp_u64<0x4E>(key);   // quad_perm [2, 3, 0, 1]
    else if constexpr (STRIDE == 8) return dpp_u64<0x128>(key);  // row_ror:8
    else if constexpr (STRIDE == 4) {
        const uint64_t below = dpp_u64<0x124>(key), above = dpp_u64<0x12C>(key);  // row_ror:4 = lane - 4, row_ror:12 = lane + 4 (mod 16)
        return (lane & 4) ? below : above;
    } else return __shfl_xor(key, STRIDE, kWave);
}

template <uint32_t STRIDE>
__device__ __forceinline__ uint64_t exchange(uint64_t key, uint32_t lane, bool keep_larger) {
    const uint64_t other = partner<STRIDE>(key, lane);
    return (key > other) == keep_larger ? key : other;
}

// The strides SIZE / 2, SIZE / 4, ..., 1 of one bitonic merge step over blocks of SIZE lanes.
template <uint32_t SIZE, uint32_t STRIDE, bool DESCENDING>
__device__ __forceinline__ uint64_t merge_strides(uint64_t key, uint32_t lane) {
    if constexpr (STRIDE == 0) return key;
    else {
        const bool block_descending = SIZE == kWave ? DESCENDING : ((lane & SIZE) == 0) == DESCENDING;
        key = exchange<STRIDE>(key, lane, ((lane & STRIDE) == 0) == block_descending);
        return merge_strides<SIZE, STRIDE / 2, DESCENDING>(key, lane);
    }
}

// Bitonic sort of one key per lane: lane i ends with the i-th largest (DESCENDING) or i-th smallest key.
template <bool DESCENDING>
__device__ __forceinline__ uint64_t wave_sort(uint64_t key, uint32_t lane) {
    key = merge_strides<2, 1, DESCENDING>(key, lane);
    key = merge_strides<4, 2, DESCENDING>(key, lane);
    key = merge_strides<8, 4, DESCENDING>(key, lane);
    key = merge_strides<16, 8, DESCENDING>(key, lane);
    key = merge_strides<32, 16, DESCENDING>(key, lane);
    return merge_strides<64, 32, DESCENDING>(key, lane);
}

// The 64 largest of a descending list and an ascending list, descending.
__device__ __forceinline__ uint64_t wave_merge(uint64_t descending, uint64_t ascending, uint32_t lane) {
    const uint64_t key = descending > ascending ? descending : ascending;
    return merge_strides<64, 32, true>(key, lane);
}

__device__ __forceinline__ uint32_t wave_min(uint32_t v) {
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
        const uint32_t o = __shfl_xor(v, m, kWave);
        v = o < v ? o : v;
    }
    return v;
}

// Merges the waves' descending lists pairwise through LDS (wave 0 ends with the workgroup's list) and writes the row.
// Every thread of the workgroup calls it (barriers inside).
__device__ void merge_waves_and_write(uint64_t top, uint64_t (*lists)[kCapacity], tsp_logit_topk_row* row, const float* logits_row,
                                      uint32_t vocabulary, uint32_t first_nonfinite, uint32_t first_subnormal) {
    const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    lists[wave][lane] = top;
    __syncthreads();
#pragma unroll
    for (uint32_t step = 1; step < kWaves; step <<= 1) {
        const bool merges = wave % (2 * step) == 0;
        if (merges) top = wave_merge(top, lists[wave + step][kWave - 1 - lane], lane);
        if (2 * step < kWaves) {
            if (merges) lists[wave][lane] = top;  // its own slot: nobody else reads it at this level
            __syncthreads();
        }
    }
    if (wave != 0) return;
    const uint32_t column = ~uint32_t(top);
    const bool live = top != 0;
    row->ids[lane] = live ? column : 0u;
    row->logits[lane] = live ? logits_row[column] : -__builtin_inff();  // the raw value, -0 included
    const uint32_t count = __builtin_popcountll(__builtin_amdgcn_ballot_w64(live));
    if (lane == 0) {
        row->vocabulary = vocabulary;
        row->count = count;
        row->first_nonfinite_col = first_nonfinite;
        row->first_subnormal_col = first_subnormal;
    }
}

__global__ __launch_bounds__(kThreads) void topk_stage1(TopKArgs a) {
    __shared__ uint64_t lists[kWaves][kCapacity];
    __shared__ uint32_t first_nonfinite, first_subnormal;
    const uint32_t tile = blockIdx.x, row = blockIdx.y, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const float* logits_row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.logits) + uint64_t(row) * a.stride_bytes);
    if (threadIdx.x == 0) { first_nonfinite = kNone; first_subnormal = kNone; }
    __syncthreads();
    uint32_t nonfinite = kNone, subnormal = kNone;
    // 4 batches of 64 columns per wave, two independent running lists so that the exchanges of one hide the other's latency
    uint64_t top[2] = {0, 0};
#pragma unroll 1
    for (uint32_t pair = 0; pair < kWaveSpan / (2 * kWave); ++pair) {
        uint64_t key[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t column = tile * kTileSpan + wave * kWaveSpan + (pair * 2 + h) * kWave + lane;
            key[h] = 0;
            if (column < a.vocabulary) {
                const float v = logits_row[column];
                const uint32_t bits = __float_as_uint(v);
                if ((bits & 0x7f800000u) == 0x7f800000u) nonfinite = nonfinite < column ? nonfinite : column;
                else if ((bits & 0x7f800000u) == 0 && (bits & 0x007fffffu) != 0) subnormal = subnormal < column ? subnormal : column;
                key[h] = make_key(v, column);
            }
        }
        if (pair == 0) {
            top[0] = wave_sort<true>(key[0], lane);
            top[1] = wave_sort<true>(key[1], lane);
        } else {
            const uint64_t c0 = wave_sort<false>(key[0], lane), c1 = wave_sort<false>(key[1], lane);
            top[0] = wave_merge(top[0], c0, lane);
            top[1] = wave_merge(top[1], c1, lane);
        }
    }
    const uint64_t mine = wave_merge(top[0], __shfl(top[1], kWave - 1 - lane, kWave), lane);
    nonfinite = wave_min(nonfinite);
    subnormal = wave_min(subnormal);
    if (lane == 0 && nonfinite != kNone) atomicMin(&first_nonfinite, nonfinite);
    if (lane == 0 && subnormal != kNone) atomicMin(&first_subnormal, subnormal);
    __syncthreads();
    const uint32_t begin = tile * kTileSpan, width = a.vocabulary - begin < kTileSpan ? a.vocabulary - begin : kTileSpan;
    merge_waves_and_write(mine, lists, a.partial + uint64_t(row) * a.tiles + tile, logits_row, width, first_nonfinite, first_subnormal);
}

__global__ __launch_bounds__(kThreads) void topk_stage2(TopKArgs a) {
    __shared__ uint64_t lists[kWaves][kCapacity];
    __shared__ uint32_t first_nonfinite, first_subnormal;
    const uint32_t row = blockIdx.x, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const float* logits_row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.logits) + uint64_t(row) * a.stride_bytes);
    const tsp_logit_topk_row* partial = a.partial + uint64_t(row) * a.tiles;
    if (threadIdx.x == 0) { first_nonfinite = kNone; first_subnormal = kNone; }
    __syncthreads();
    // a partial row is a descending list (empty slots have key 0); read backwards it is ascending
    auto list_key = [&](uint32_t tile, uint32_t slot) -> uint64_t {
        return tile < a.tiles && slot < partial[tile].count ? make_key(partial[tile].logits[slot], partial[tile].ids[slot]) : 0;
    };
    uint64_t top[2] = {list_key(wave, lane), list_key(wave + kWaves, lane)};
#pragma unroll 1
    for (uint32_t tile = wave + 2 * kWaves; tile < a.tiles; tile += 2 * kWaves) {  // a pair per round; a tile past the end is an empty list
        const uint64_t c0 = list_key(tile, kWave - 1 - lane), c1 = list_key(tile + kWaves, kWave - 1 - lane);
        top[0] = wave_merge(top[0], c0, lane);
        top[1] = wave_merge(top[1], c1, lane);
    }
    const uint64_t mine = wave_merge(top[0], __shfl(top[1], kWave - 1 - lane, kWave), lane);
    for (uint32_t tile = threadIdx.x; tile < a.tiles; tile += blockDim.x) {
        if (partial[tile].first_nonfinite_col != kNone) atomicMin(&first_nonfinite, partial[tile].first_nonfinite_col);
        if (partial[tile].first_subnormal_col != kNone) atomicMin(&first_subnormal, partial[tile].first_subnormal_col);
    }
    __syncthreads();
    merge_waves_and_write(mine, lists, a.out + row, logits_row, a.vocabulary, first_nonfinite, first_subnormal);
}

uint32_t tiles_for(uint32_t vocabulary) { return (vocabulary + kTileSpan - 1) / kTileSpan; }

int launch_topk(const TopKArgs& a, hipStream_t s) {
    TSP_LAUNCH("logit_topk_stage1", s, topk_stage1<<<dim3(a.tiles, a.rows), kThreads, 0, s>>>(a));
    const int rc = launch_status("logit_topk_stage1");
    if (rc != TSP_OK) return rc;
    TSP_LAUNCH("logit_topk_stage2", s, topk_stage2<<<a.rows, kThreads, 0, s>>>(a));
    return launch_status("logit_topk_stage2");
}

}  // namespace

extern "C" uint64_t tsp_logit_topk_scratch_bytes(uint32_t max_rows, uint32_t max_vocabulary) {
    if (max_rows < 1 || max_rows > 2048 || max_vocabulary < 1 || max_vocabulary > (1u << 20)) {
        set_error("GPU logit top-k scratch bounds mismatch");
        return 0;
    }
    const uint32_t tiles = tiles_for(max_vocabulary) < kMaxTiles ? tiles_for(max_vocabulary) : kMaxTiles;
    return uint64_t(max_rows) * tiles * sizeof(tsp_logit_topk_row);
}

extern "C" uint64_t tsp_logit_topk_output_bytes(uint32_t max_rows) {
    if (max_rows < 1 || max_rows > 2048) {
        set_error("GPU logit top-k output row count out of bounds");
        return 0;
    }
    return uint64_t(max_rows) * sizeof(tsp_logit_topk_row);
}

extern "C" int tsp_logit_topk(const float* logits, uint64_t stride_bytes, uint32_t rows, uint32_t vocabulary, void* partial_scratch,
                              uint64_t scratch_bytes, void* out_rows, uint64_t out_bytes, void* stream) {
    static_assert(sizeof(tsp_logit_topk_row) == 528, "top-k row ABI");
    TSP_REQUIRE(rows >= 1 && rows <= 2048 && vocabulary >= 1 && vocabulary <= (1u << 20) && stride_bytes >= uint64_t(vocabulary) * 4 &&
                    stride_bytes % 4 == 0,
                "GPU logit top-k geometry mismatch");
    const uint32_t tiles = tiles_for(vocabulary);
    TSP_REQUIRE(tiles >= 1 && tiles <= kMaxTiles, "GPU logit top-k tile count out of bounds");
    TSP_REQUIRE(logits && partial_scratch && out_rows, "null device pointer");
    const uint64_t in_bytes = uint64_t(rows - 1) * stride_bytes + uint64_t(vocabulary) * 4;
    const uint64_t need_scratch = uint64_t(rows) * tiles * sizeof(tsp_logit_topk_row), need_out = uint64_t(rows) * sizeof(tsp_logit_topk_row);
    TSP_REQUIRE(scratch_bytes >= need_scratch && out_bytes >= need_out && reinterpret_cast<uintptr_t>(logits) % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(partial_scratch) % 4 == 0 && reinterpret_cast<uintptr_t>(out_rows) % 4 == 0,
                "GPU logit top-k buffer span or alignment mismatch");
    TSP_REQUIRE(!ranges_overlap(logits, in_bytes, partial_scratch, need_scratch) && !ranges_overlap(logits, in_bytes, out_rows, need_out) &&
                    !ranges_overlap(partial_scratch, need_scratch, out_rows, need_out),
                "GPU logit top-k buffers overlap");
    TopKArgs a{logits, stride_bytes, rows, vocabulary, tiles, static_cast<tsp_logit_topk_row*>(partial_scratch),
               static_cast<tsp_logit_topk_row*>(out_rows)};
    return launch_topk(a, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------- the same operator for callers that cannot allocate
// The partial rows live in a file-scope device array instead of a caller's buffer. In host code the array's name is only
// a handle: its device address is asked for once per device (each device holds its own copy at its own address) and kept.
namespace {
constexpr uint32_t kStaticRows = 16, kStaticTiles = 64;  // 16 rows x 262 144 columns: 540 672 bytes per device
}
static __device__ __align__(256) uint8_t scratch[uint64_t(kStaticRows) * kStaticTiles * sizeof(tsp_logit_topk_row)];
namespace {
std::atomic<void*> g_scratch_at[64];
int static_scratch(void** at) {
    int device = 0;
    TSP_HIP(hipGetDevice(&device));
    TSP_REQUIRE(device >= 0 && device < 64, "GPU logit top-k: device ordinal out of range");
    void* p = g_scratch_at[device].load(std::memory_order_acquire);
    if (!p) {
        TSP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        TSP_REQUIRE(p != nullptr, "GPU logit top-k: the static scratch array has no device address");
        g_scratch_at[device].store(p, std::memory_order_release);
    }
    *at = p;
    return TSP_OK;
}
}  // namespace

static_assert(kStaticRows == TSP_LOGIT_TOPK_STATIC_MAX_ROWS && kStaticTiles * kTileSpan == TSP_LOGIT_TOPK_STATIC_MAX_VOCABULARY, "limits in the header");

extern "C" int tsp_logit_topk_static(const float* logits, uint64_t stride_bytes, uint32_t rows, uint32_t vocabulary, void* out_rows,
                                     uint64_t out_bytes, void* stream) {
    TSP_REQUIRE(rows >= 1 && rows <= kStaticRows && vocabulary >= 1 && vocabulary <= kStaticTiles * kTileSpan,
                "GPU logit top-k without a scratch argument takes at most %u rows of at most %u columns", kStaticRows, kStaticTiles * kTileSpan);
    TSP_REQUIRE(stride_bytes >= uint64_t(vocabulary) * 4 && stride_bytes % 4 == 0, "GPU logit top-k geometry mismatch");
    TSP_REQUIRE(logits && out_rows, "null device pointer");
    const uint32_t tiles = tiles_for(vocabulary);
    const uint64_t in_bytes = uint64_t(rows - 1) * stride_bytes + uint64_t(vocabulary) * 4, need_out = uint64_t(rows) * sizeof(tsp_logit_topk_row);
    TSP_REQUIRE(out_bytes >= need_out && reinterpret_cast<uintptr_t>(logits) % 4 == 0 && reinterpret_cast<uintptr_t>(out_rows) % 4 == 0,
                "GPU logit top-k buffer span or alignment mismatch");
    TSP_REQUIRE(!ranges_overlap(logits, in_bytes, out_rows, need_out), "GPU logit top-k buffers overlap");
    void* partial = nullptr;
    const int rc = static_scratch(&partial);
    if (rc != TSP_OK) return rc;
    // every partial row stage 2 reads is written by stage 1 of the same call: nothing has to start at zero
    TopKArgs a{logits, stride_bytes, rows, vocabulary, tiles, static_cast<tsp_logit_topk_row*>(partial), static_cast<tsp_logit_topk_row*>(out_rows)};
    return launch_topk(a, static_cast<hipStream_t>(stream));
}
