// The router projection of a prefill chunk as one f32 GEMM: logits[token, expert] = sum_k W[expert, k] * x[token, k].
//
// Replaces the engine's `graph_moe_router_f32_batch` (kernels/moe_router_f32_batch.metal:13-50: 32x32x32 f32 tiles,
// full-precision multiply-accumulate, operands never narrowed) and its windowed sibling for up to 2048 tokens.
// Both operands stay f32 from memory to the accumulator: the products run on the f32 matrix-core instruction
// (v_mfma_f32_32x32x2_f32), which rounds once per fused multiply-add like the scalar code does.
//
// One workgroup of eight waves owns a 64 token x 64 expert tile. Per 64-column step both 64 x 64 operand tiles go
// global -> registers -> LDS (rows padded to 68 floats so that the 16-byte fragment reads of a wave spread over all
// banks), double buffered with one barrier per step; waves 0-3 multiply the first 32 columns of the step, waves 4-7 the
// last 32, so every SIMD holds two waves that hide each other's LDS latency. The two halves are added in a fixed order
// at the end (deterministic). Consecutive tiles of one token block go to one XCD so that its L2 serves the x rows.
#include "tsp_common.hpp"

using namespace tsp;

namespace {

constexpr uint32_t kTile = 64;                          // tokens and experts per workgroup
constexpr uint32_t kStep = 64;                          // columns per LDS stage
constexpr uint32_t kPitch = 68;                         // floats per LDS row
constexpr uint32_t kStageFloats = 2 * kTile * kPitch;   // x tile, then W tile
constexpr uint32_t kLdsBytes = 2 * kStageFloats * 4;    // 69 632

typedef float acc16 __attribute__((ext_vector_type(16)));

struct RouterArgs {
    const float* weights;
    const float* input;
    float* output;
    uint64_t input_stride, output_stride;  // floats
    uint32_t columns, experts, tokens;
    uint32_t expert_tiles, tiles, tiles_per_xcd;
    uint32_t* error_word;
};

__global__ __launch_bounds__(512) void router_f32_gemm(RouterArgs a) {
    extern __shared__ __align__(16) float lds[];
    // blockIdx % 8 names the XCD; each XCD takes a contiguous run of tiles (all expert tiles of a token block together)
    const uint32_t tile = (blockIdx.x % 8) * a.tiles_per_xcd + blockIdx.x / 8;
    if (tile >= a.tiles || blockIdx.x / 8 >= a.tiles_per_xcd) return;
    const uint32_t token0 = (tile / a.expert_tiles) * kTile, expert0 = (tile % a.expert_tiles) * kTile;
    const uint32_t tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const uint32_t half = wave / 4, wt = (wave % 4) / 2, we = wave % 2;

    // staging: thread t moves float4 number t and t + 512 of each 64 x 64 tile (row = n / 16, 16-byte column = n % 16)
    const float* xrow[2];
    const float* wrow[2];
    uint32_t slot[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t n = tid + i * 512, row = n / 16, c4 = n % 16;
        const uint32_t token = min(token0 + row, a.tokens - 1), expert = min(expert0 + row, a.experts - 1);  // tails re-read a valid row
        xrow[i] = a.input + uint64_t(token) * a.input_stride + c4 * 4;
        wrow[i] = a.weights + uint64_t(expert) * a.columns + c4 * 4;
        slot[i] = row * kPitch + c4 * 4;
    }
    const uint32_t c4 = tid % 16;
    float4 rx[2], rw[2];
    auto fetch = [&](uint32_t step) {
        const uint32_t k = step * kStep;
        const bool inside = k + c4 * 4 < a.columns;  // columns is a multiple of 32: a last half step reads zeros
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            rx[i] = inside ? *reinterpret_cast<const float4*>(xrow[i] + k) : float4{0, 0, 0, 0};
            rw[i] = inside ? *reinterpret_cast<const float4*>(wrow[i] + k) : float4{0, 0, 0, 0};
        }
    };
    auto stash = [&](uint32_t stage) {
        float* base = lds + stage * kStageFloats;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<float4*>(base + slot[i]) = rx[i];
            *reinterpret_cast<float4*>(base + kTile * kPitch + slot[i]) = rw[i];
        }
    };

    // fragments of v_mfma_f32_32x32x2_f32: lane holds A[lane % 32][lane / 32] and B[lane / 32][lane % 32]. A 16-byte read
    // gives a lane four columns; the same four go to A and B, so the order in which columns meet does not matter.
    const uint32_t frag_x = (wt * 32 + lane % 32) * kPitch + half * 32 + (lane / 32) * 4;
    const uint32_t frag_w = kTile * kPitch + (we * 32 + lane % 32) * kPitch + half * 32 + (lane / 32) * 4;
    acc16 acc = {};
    const uint32_t steps = (a.columns + kStep - 1) / kStep;
    fetch(0);
    stash(0);
    if (steps > 1) fetch(1);
    __syncthreads();
    for (uint32_t s = 0; s < steps; ++s) {
        const float* base = lds + (s & 1) * kStageFloats;
        float4 fx[4], fw[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            fx[q] = *reinterpret_cast<const float4*>(base + frag_x + q * 8);
            fw[q] = *reinterpret_cast<const float4*>(base + frag_w + q * 8);
        }
        if (s + 1 < steps) stash((s + 1) & 1);   // the other stage: every wave left it before the last barrier
        if (s + 2 < steps) fetch(s + 2);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[q].x, fw[q].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[q].y, fw[q].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[q].z, fw[q].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fx[q].w, fw[q].w, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // second column half -> LDS -> added by the wave that owns the same 32 x 32 block
    float* sums = lds + (wave % 4) * 1024;
    if (half == 1) {
#pragma unroll
        for (int v = 0; v < 16; ++v) sums[v * 64 + lane] = acc[v];
    }
    __syncthreads();
    if (half == 0) {
        uint32_t bad = 0;
        const uint32_t expert = expert0 + we * 32 + lane % 32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float value = acc[v] + sums[v * 64 + lane];
            const uint32_t token = token0 + wt * 32 + (v / 4) * 8 + (lane / 32) * 4 + v % 4;  // D[i][j]: j = lane % 32
            if (token < a.tokens && expert < a.experts) {
                bad |= nonfinite(value) ? TSP_ERRBIT_NONFINITE : 0u;
                a.output[uint64_t(token) * a.output_stride + expert] = value;
            }
        }
        publish_error(bad, a.error_word);
    }
}

std::atomic<uint64_t> g_lds_raised{0};

}  // namespace

extern "C" int tsp_router_f32_batch(const float* weights, const float* input, uint64_t input_stride_bytes, float* output,
                                    uint64_t output_stride_bytes, uint32_t columns, uint32_t experts, uint32_t tokens,
                                    uint32_t* error_word, void* stream) {
    TSP_REQUIRE(weights && input && output && error_word, "null device pointer");
    TSP_REQUIRE(columns && columns % 32 == 0 && columns <= 65536 && experts && experts <= 65536 && tokens && tokens <= 65536,
                "router f32 batch geometry (columns in multiples of 32)");
    TSP_REQUIRE(input_stride_bytes >= uint64_t(columns) * 4 && output_stride_bytes >= uint64_t(experts) * 4 && input_stride_bytes % 16 == 0 &&
                    output_stride_bytes % 16 == 0 && input_stride_bytes <= (1ull << 32) && output_stride_bytes <= (1ull << 32),
                "router f32 batch stride");
    TSP_REQUIRE(reinterpret_cast<uintptr_t>(weights) % 16 == 0 && reinterpret_cast<uintptr_t>(input) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(output) % 4 == 0,
                "router f32 batch alignment (16 bytes for the operands)");
    const uint64_t in_span = uint64_t(tokens - 1) * input_stride_bytes + uint64_t(columns) * 4;
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(experts) * 4;
    const uint64_t w_span = uint64_t(columns) * experts * 4;
    TSP_REQUIRE(!ranges_overlap(output, out_span, input, in_span) && !ranges_overlap(output, out_span, weights, w_span),
                "router f32 batch output overlaps an input");
    int device = 0;
    if (setup_pending(g_lds_raised, &device)) {
        TSP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(router_f32_gemm), hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytes)));
        setup_done(g_lds_raised, device);
    }
    RouterArgs a{};
    a.weights = weights; a.input = input; a.output = output;
    a.input_stride = input_stride_bytes / 4; a.output_stride = output_stride_bytes / 4;
    a.columns = columns; a.experts = experts; a.tokens = tokens;
    a.expert_tiles = (experts + kTile - 1) / kTile;
    a.tiles = a.expert_tiles * ((tokens + kTile - 1) / kTile);
    a.tiles_per_xcd = (a.tiles + 7) / 8;
    a.error_word = error_word;
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("router_f32_gemm", s, router_f32_gemm<<<a.tiles_per_xcd * 8, 512, kLdsBytes, s>>>(a));
    return launch_status("router_f32_gemm");
}
