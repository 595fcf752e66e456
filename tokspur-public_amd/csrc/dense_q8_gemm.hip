// Dense Q8_0 GEMM for many token rows (the shared expert of a prefill chunk): out[t, n] = sum_k x[t, k] * d[n, k/32] * q[n, k].
//
// The streaming kernels of q8.hip / q8_mfma.hip read the whole matrix once per 8 or 16 token rows: right for decode,
// hundreds of passes for a 2048-token chunk. Here the matrix is decoded once per call into halves (d * q rounded to
// nearest: 11 significant bits, what the engine's own kernel stages, include/tokspur/graph.hpp:860 and
// kernels/grouped_mm.metal:239-243), the token rows are rounded to halves as well, and one matrix-core GEMM with f32
// accumulation multiplies the two. Both operands are K-contiguous rows, so the GEMM is the "NT" form and both tiles are
// staged the same way.
//
// GEMM kernel: a workgroup of four waves owns a 64 x 64 output tile (each wave a 32 x 32 MFMA tile) and walks K in
// steps of 64 halfs. Every byte travels global -> LDS directly (16 bytes per lane, no registers in between) into a ring
// of four stages, three steps ahead of the multiply; chunk c of row r of a slab sits at position r * 8 + (c ^ (r & 7)),
// which the loads fill linearly by lane and the fragment reads spread over all banks. No other vector-memory operation
// exists in the loop, so the wait before a step's barrier is simply "all but the two younger stages have landed".
#include "mfma_quant.hpp"

using namespace tsp;

namespace {

constexpr int kTile = 64, kStep = 64;                  // output tile edge; halfs of K per step (128 B per row)
constexpr int kSlabBytes = kTile * kStep * 2;          // 8 KB: 64 rows x 128 B
constexpr int kStageBytes = 2 * kSlabBytes;            // token slab, weight slab
constexpr int kRing = 4;

struct F16GemmArgs {
    const _Float16* x;  // [m][k]
    const _Float16* w;  // [n][k]
    float* out;         // rows out_stride bytes apart
    uint64_t out_stride;
    uint32_t m, n, k;
    uint32_t* error_word;
};

__global__ __launch_bounds__(256, 2) void f16_gemm_nt(F16GemmArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kRing * kStageBytes];  // 64 KB: two workgroups per CU
    const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const uint32_t col = lane % 32, khalf = lane / 32;
    const uint32_t m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
    const uint32_t steps = a.k / kStep;

    // piece p = i * 256 + tid of a stage (1024 pieces of 16 bytes): slab p / 512, LDS position q = p % 512 -> row q / 8,
    // chunk (q % 8) ^ (row & 7). Rows past the matrix re-read its last row (never stored).
    const uint8_t* src[4];
    uint32_t lds_at[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t p = i * 256 + tid, slab = p / 512, q = p % 512, r = q / 8, c = (q % 8) ^ (r & 7);
        uint32_t row = (slab ? n0 : m0) + r;
        const uint32_t limit = slab ? a.n : a.m;
        row = row < limit ? row : limit - 1;
        src[i] = reinterpret_cast<const uint8_t*>(slab ? a.w : a.x) + (uint64_t(row) * a.k + c * 8) * 2;
        lds_at[i] = __builtin_amdgcn_readfirstlane(lds_address(lds) + (i * 256 + wave * kWave) * 16);  // lane 0 of this wave; the hardware adds 16 * lane
    }
    auto request = [&](uint32_t step, uint32_t slot) {  // steps past the end re-read the last one into a slot nobody reads
        const uint32_t s = step < steps ? step : steps - 1;
#pragma unroll
        for (int i = 0; i < 4; ++i) load_to_lds_16(src[i] + uint64_t(s) * kStep * 2, lds_at[i] + slot * kStageBytes);
    };

    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    const uint32_t arow = (wave / 2) * 32 + col, brow = (wave % 2) * 32 + col;
    request(0, 0);
    request(1, 1);
    request(2, 2);
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t slot = s % kRing;
        lds_barrier_after_loads<8>();  // stage s has landed (the two younger stages may be on their way); every wave has left slot (s + 3) % 4
        request(s + 3, (s + 3) % kRing);
        const uint8_t* xs = lds + slot * kStageBytes;
        const uint8_t* ws = xs + kSlabBytes;
#pragma unroll
        for (int kc = 0; kc < 4; ++kc) {
            const uint32_t c = kc * 2 + khalf;
            const f16x8 fa = *reinterpret_cast<const f16x8*>(xs + (arow * 8 + (c ^ (arow & 7))) * 16);
            const f16x8 fb = *reinterpret_cast<const f16x8*>(ws + (brow * 8 + (c ^ (brow & 7))) * 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc, 0, 0, 0);
        }
    }
    wait_all_loads();  // the last requests land in slots nobody reads: they must be done before this LDS is given away

    // accumulator v: token row 8 * (v / 4) + 4 * khalf + v % 4 of the wave's tile, weight row `col`
    uint32_t bad = 0;
    const uint32_t n = n0 + (wave % 2) * 32 + col;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const uint32_t m = m0 + (wave / 2) * 32 + 8 * (v / 4) + 4 * khalf + (v % 4);
        if (m < a.m && n < a.n) {
            if (nonfinite(acc[v])) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.out) + uint64_t(m) * a.out_stride)[n] = acc[v];
        }
    }
    publish_error(bad, a.error_word);
}

// Two weights per thread: GGUF rows are 34-byte blocks (f16 d, 32 int8); q8_lanes_v1 rows keep the scales first, then runs
// of 16 blocks with byte = index * width + block % 16 (src/expert_lanes.cpp:60-119).
__global__ __launch_bounds__(256) void q8_rows_to_f16(const uint8_t* __restrict__ matrix, uint32_t layout, _Float16* __restrict__ out,
                                                      uint32_t columns, uint32_t rows) {
    const uint64_t pair = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (pair >= uint64_t(rows) * (columns / 2)) return;
    const uint32_t row = uint32_t(pair / (columns / 2)), c = uint32_t(pair % (columns / 2)) * 2;
    const uint32_t blocks = columns / 32, block = c / 32, index = c % 32;
    const uint8_t* data = matrix + uint64_t(row) * blocks * 34;
    float d;
    int q0, q1;
    if (layout == TSP_LAYOUT_GGUF) {
        const uint8_t* b = data + block * 34;
        d = half_bits_to_float(uint32_t(b[0]) | (uint32_t(b[1]) << 8));
        q0 = int(int8_t(b[2 + index]));
        q1 = int(int8_t(b[3 + index]));
    } else {
        const uint32_t run = block / 16, width = blocks - run * 16 < 16 ? blocks - run * 16 : 16;
        const uint8_t* q = data + blocks * 2 + run * 512 + block % 16;
        d = half_bits_to_float(uint32_t(data[block * 2]) | (uint32_t(data[block * 2 + 1]) << 8));
        q0 = int(int8_t(q[index * width]));
        q1 = int(int8_t(q[(index + 1) * width]));
    }
    const f16x2 pairs{_Float16(d * float(q0)), _Float16(d * float(q1))};  // d * q is exact in f32: one rounding
    *reinterpret_cast<f16x2*>(out + uint64_t(row) * columns + c) = pairs;
}

// Eight values per thread; a value that does not fit a half (or is not finite) raises the non-finite bit.
__global__ __launch_bounds__(256) void f32_rows_to_f16(const float* __restrict__ x, uint64_t stride_bytes, _Float16* __restrict__ out,
                                                       uint32_t rows, uint32_t columns, uint32_t* error_word) {
    const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    uint32_t bad = 0;
    if (i < uint64_t(rows) * (columns / 8)) {
        const uint32_t r = uint32_t(i / (columns / 8)), c8 = uint32_t(i % (columns / 8));
        const float* src = reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(x) + uint64_t(r) * stride_bytes) + c8 * 8;
        f16x8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            h[e] = _Float16(src[e]);
            if ((__builtin_bit_cast(uint16_t, h[e]) & 0x7c00u) == 0x7c00u) bad = TSP_ERRBIT_NONFINITE;
        }
        *reinterpret_cast<f16x8*>(out + uint64_t(r) * columns + c8 * 8) = h;
    }
    publish_error(bad, error_word);
}

uint64_t align256(uint64_t v) { return (v + 255) / 256 * 256; }

}  // namespace

// workspace: [decoded matrix, halves][token rows, halves]
extern "C" uint64_t tsp_dense_mm_q8_workspace_bytes(uint32_t tokens, uint32_t columns, uint32_t rows) {
    return align256(uint64_t(rows) * columns * 2) + align256(uint64_t(tokens) * columns * 2);
}

extern "C" int tsp_dense_mm_q8_staged(uint32_t layout, const void* matrix, uint64_t matrix_bytes, const float* input, uint64_t input_stride_bytes,
                                      float* output, uint64_t output_stride_bytes, uint32_t tokens, uint32_t columns, uint32_t rows,
                                      void* workspace, uint64_t workspace_bytes, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(layout == TSP_LAYOUT_GGUF || layout == TSP_LAYOUT_Q8_LANES_V1, "dense Q8_0 GEMM layout");
    TSP_REQUIRE(columns && columns <= 65536 && columns % 64 == 0 && rows && rows <= 1000000 && tokens && tokens <= 65536,
                "staged dense Q8_0 GEMM needs columns in multiples of 64");
    TSP_REQUIRE(uint64_t(columns / 32) * rows * 34 == matrix_bytes, "dense Q8_0 GEMM matrix byte span mismatch");
    TSP_REQUIRE(input_stride_bytes % 4 == 0 && output_stride_bytes % 4 == 0 && input_stride_bytes >= uint64_t(columns) * 4 &&
                    output_stride_bytes >= uint64_t(rows) * 4,
                "dense Q8_0 GEMM row geometry mismatch");
    TSP_REQUIRE(matrix && input && output && workspace && error_word, "null device pointer");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && workspace_bytes >= tsp_dense_mm_q8_workspace_bytes(tokens, columns, rows),
                "dense Q8_0 GEMM workspace too small or misaligned");
    const uint64_t in_span = uint64_t(tokens - 1) * input_stride_bytes + uint64_t(columns) * 4;
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(rows) * 4;
    TSP_REQUIRE(!ranges_overlap(output, out_span, matrix, matrix_bytes) && !ranges_overlap(output, out_span, input, in_span) &&
                    !ranges_overlap(workspace, workspace_bytes, matrix, matrix_bytes) && !ranges_overlap(workspace, workspace_bytes, input, in_span) &&
                    !ranges_overlap(workspace, workspace_bytes, output, out_span),
                "dense Q8_0 GEMM buffers overlap");
    const auto s = static_cast<hipStream_t>(stream);
    _Float16* const w16 = static_cast<_Float16*>(workspace);
    _Float16* const x16 = reinterpret_cast<_Float16*>(static_cast<uint8_t*>(workspace) + align256(uint64_t(rows) * columns * 2));
    const uint64_t pairs = uint64_t(rows) * (columns / 2), eights = uint64_t(tokens) * (columns / 8);
    TSP_LAUNCH("q8_rows_to_f16", s, q8_rows_to_f16<<<uint32_t((pairs + 255) / 256), 256, 0, s>>>(static_cast<const uint8_t*>(matrix), layout, w16, columns, rows));
    TSP_LAUNCH("f32_rows_to_f16", s, f32_rows_to_f16<<<uint32_t((eights + 255) / 256), 256, 0, s>>>(input, input_stride_bytes, x16, tokens, columns, error_word));
    const F16GemmArgs a{x16, w16, output, output_stride_bytes, tokens, rows, columns, error_word};
    const dim3 grid((rows + kTile - 1) / kTile, (tokens + kTile - 1) / kTile);
    TSP_LAUNCH("f16_gemm_nt", s, f16_gemm_nt<<<grid, 256, 0, s>>>(a));
    return launch_status("f16_gemm_nt");
}
