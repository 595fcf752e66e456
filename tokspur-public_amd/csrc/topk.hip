// Row top-64 of a logits matrix: for every row the 64 largest finite logits in the order
// (value descending, column ascending, -0 == +0), the number found, and the first non-finite and first
// subnormal column. Rank 0 is the arg-max a greedy sampler needs.
//
// Two launches. Stage 1: one workgroup per (4096-column tile, row) sorts its tile and writes a partial row.
// Stage 2: one workgroup per row sorts the partial rows' candidates and writes the final row. Both stages sort
// 64-bit keys with a bitonic network in LDS: high word = the float mapped to an unsigned integer of the same
// order (after -0 -> +0), low word = ~column, so that "largest key first" is exactly the ordering above.
// Non-finite logits and padding get key 0, below every finite value's key.
#include "tsp_common.hpp"

using namespace tsp;

namespace {

constexpr uint32_t kCapacity = 64, kTileSpan = 4096, kMaxTiles = 256, kNone = 0xffffffffu;

struct TopKArgs {
    const float* logits;
    uint64_t stride_bytes;
    uint32_t rows, vocabulary, tiles;
    tsp_logit_topk_row* partial;  // [rows][tiles]
    tsp_logit_topk_row* out;      // [rows]
    uint32_t sort_size;           // stage 2: power of two >= tiles * 64
};

__device__ __forceinline__ uint64_t make_key(float value, uint32_t column) {
    uint32_t bits = __float_as_uint(value);
    if ((bits & 0x7f800000u) == 0x7f800000u) return 0;  // inf / nan never rank
    if ((bits & 0x7fffffffu) == 0) bits = 0;             // -0 ranks as +0
    const uint32_t ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return (uint64_t(ordered) << 32) | uint32_t(~column);
}

// Descending bitonic sort of `n` (a power of two) keys in LDS by the whole workgroup.
__device__ void sort_descending(uint64_t* keys, uint32_t n) {
    for (uint32_t size = 2; size <= n; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (uint32_t t = threadIdx.x; t < n / 2; t += blockDim.x) {
                const uint32_t lo = 2 * t - (t & (stride - 1)), hi = lo + stride;
                const bool descending = (lo & size) == 0;
                const uint64_t a = keys[lo], b = keys[hi];
                if ((a < b) == descending) { keys[lo] = b; keys[hi] = a; }
            }
        }
    }
    __syncthreads();
}

__device__ void write_row(tsp_logit_topk_row* row, const uint64_t* keys, const float* logits_row, uint32_t vocabulary,
                          uint32_t first_nonfinite, uint32_t first_subnormal) {
    if (threadIdx.x < kCapacity) {
        const uint64_t key = keys[threadIdx.x];
        const uint32_t column = ~uint32_t(key);
        const bool live = key != 0;
        row->ids[threadIdx.x] = live ? column : 0u;
        row->logits[threadIdx.x] = live ? logits_row[column] : -__builtin_inff();  // the raw value, -0 included
    }
    if (threadIdx.x == 0) {
        uint32_t count = 0;
        while (count < kCapacity && keys[count] != 0) ++count;
        row->vocabulary = vocabulary;
        row->count = count;
        row->first_nonfinite_col = first_nonfinite;
        row->first_subnormal_col = first_subnormal;
    }
}

__global__ __launch_bounds__(256) void topk_stage1(TopKArgs a) {
    __shared__ uint64_t keys[kTileSpan];
    __shared__ uint32_t first_nonfinite, first_subnormal;
    const uint32_t tile = blockIdx.x, row = blockIdx.y;
    const float* logits_row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.logits) + uint64_t(row) * a.stride_bytes);
    if (threadIdx.x == 0) { first_nonfinite = kNone; first_subnormal = kNone; }
    __syncthreads();
    uint32_t nonfinite = kNone, subnormal = kNone;
    for (uint32_t i = threadIdx.x; i < kTileSpan; i += blockDim.x) {
        const uint32_t column = tile * kTileSpan + i;
        uint64_t key = 0;
        if (column < a.vocabulary) {
            const float v = logits_row[column];
            const uint32_t bits = __float_as_uint(v);
            if ((bits & 0x7f800000u) == 0x7f800000u) nonfinite = nonfinite < column ? nonfinite : column;
            else if ((bits & 0x7f800000u) == 0 && (bits & 0x007fffffu) != 0) subnormal = subnormal < column ? subnormal : column;
            key = make_key(v, column);
        }
        keys[i] = key;
    }
    if (nonfinite != kNone) atomicMin(&first_nonfinite, nonfinite);
    if (subnormal != kNone) atomicMin(&first_subnormal, subnormal);
    sort_descending(keys, kTileSpan);
    const uint32_t begin = tile * kTileSpan, width = a.vocabulary - begin < kTileSpan ? a.vocabulary - begin : kTileSpan;
    write_row(a.partial + uint64_t(row) * a.tiles + tile, keys, logits_row, width, first_nonfinite, first_subnormal);
}

__global__ __launch_bounds__(256) void topk_stage2(TopKArgs a) {
    extern __shared__ uint64_t merged[];
    __shared__ uint32_t first_nonfinite, first_subnormal;
    const uint32_t row = blockIdx.x;
    const float* logits_row = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(a.logits) + uint64_t(row) * a.stride_bytes);
    const tsp_logit_topk_row* partial = a.partial + uint64_t(row) * a.tiles;
    if (threadIdx.x == 0) { first_nonfinite = kNone; first_subnormal = kNone; }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < a.sort_size; i += blockDim.x) {
        const uint32_t tile = i / kCapacity, slot = i % kCapacity;
        uint64_t key = 0;
        if (tile < a.tiles && slot < partial[tile].count) key = make_key(partial[tile].logits[slot], partial[tile].ids[slot]);
        merged[i] = key;
    }
    for (uint32_t tile = threadIdx.x; tile < a.tiles; tile += blockDim.x) {
        if (partial[tile].first_nonfinite_col != kNone) atomicMin(&first_nonfinite, partial[tile].first_nonfinite_col);
        if (partial[tile].first_subnormal_col != kNone) atomicMin(&first_subnormal, partial[tile].first_subnormal_col);
    }
    sort_descending(merged, a.sort_size);
    write_row(a.out + row, merged, logits_row, a.vocabulary, first_nonfinite, first_subnormal);
}

uint32_t tiles_for(uint32_t vocabulary) { return (vocabulary + kTileSpan - 1) / kTileSpan; }

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
               static_cast<tsp_logit_topk_row*>(out_rows), 64};
    while (a.sort_size < tiles * kCapacity) a.sort_size <<= 1;
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("logit_topk_stage1", s, topk_stage1<<<dim3(tiles, rows), 256, 0, s>>>(a));
    int rc = launch_status("logit_topk_stage1");
    if (rc != TSP_OK) return rc;
    const uint32_t lds_bytes = a.sort_size * 8;
    static bool raised = false;
    if (lds_bytes > 48 * 1024 && !raised) {
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&topk_stage2), hipFuncAttributeMaxDynamicSharedMemorySize, kMaxTiles * kCapacity * 8));
        raised = true;
    }
    TSP_LAUNCH("logit_topk_stage2", s, topk_stage2<<<rows, 256, lds_bytes, s>>>(a));
    return launch_status("logit_topk_stage2");
}
