// Router top-k with softmax / sigmoid weights, the weighted mixture (combine) and SwiGLU.
//
// Top-k is integer-exact: k rounds of arg-max over f32 logits compared as given (as 32-bit integers of
// the same order), exact ties to the lower expert id. One 64-lane wave owns one token row and keeps the row's logits in registers
// (lane i holds experts i, i+64, ...), so a round is a per-lane scan plus two wave reductions and
// no barrier. Weights use accurate expf/logf; their association differs from a sequential sum but
// they are compared to the double reference under tolerance, never bit for bit.
#include "tsp_common.hpp"

using namespace tsp;

namespace {

__device__ __forceinline__ float sigmoid_f(float x) {
    if (x >= 0) return 1.0f / (1.0f + expf(-x));
    const float e = expf(x);
    return e / (1.0f + e);
}

__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ float route_activation(float logit, float maximum, uint32_t mode, uint32_t normalize) {
    if (!mode) return expf(logit - maximum);
    if (normalize) return expf(-softplus_f(-logit) + softplus_f(-maximum));
    return sigmoid_f(logit);
}

// A logit as an unsigned integer of the same order (-0 as +0). Every finite or infinite logit maps above 0, so 0 = no candidate.
__device__ __forceinline__ uint32_t ordered_logit(float logit) {
    uint32_t bits = __float_as_uint(logit);
    if ((bits & 0x7fffffffu) == 0) bits = 0;
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
__device__ __forceinline__ float logit_of_ordered(uint32_t ordered) {
    return __uint_as_float((ordered & 0x80000000u) ? (ordered & 0x7fffffffu) : ~ordered);
}
// Four cross-lane steps inside each row of 16 lanes leave the row's result in all its lanes; the four rows meet in scalar registers.
template <int Ctrl, bool MAX>
__device__ __forceinline__ uint32_t dpp_step_u32(uint32_t v) {
    const uint32_t other = uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), Ctrl, 0xf, 0xf, false));
    return MAX ? (other > v ? other : v) : (other < v ? other : v);
}
template <bool MAX>
__device__ __forceinline__ uint32_t wave_extreme_u32(uint32_t v) {
    v = dpp_step_u32<0xB1, MAX>(v);   // quad_perm [1,0,3,2]
    v = dpp_step_u32<0x4E, MAX>(v);   // quad_perm [2,3,0,1]
    v = dpp_step_u32<0x141, MAX>(v);  // row_half_mirror
    v = dpp_step_u32<0x140, MAX>(v);  // row_mirror
    uint32_t best = uint32_t(__builtin_amdgcn_readlane(int(v), 0));
#pragma unroll
    for (int row = 1; row < 4; ++row) {
        const uint32_t r = uint32_t(__builtin_amdgcn_readlane(int(v), row * 16));
        best = MAX ? (r > best ? r : best) : (r < best ? r : best);
    }
    return best;
}
__device__ __forceinline__ float wave_sum_shfl(float v) {
    for (int m = 1; m < kWave; m <<= 1) v += __shfl_xor(v, m, kWave);
    return v;
}

// CAND = ceil(experts / 64) register slots per lane (8 covers 512 experts, 64 covers 4096).
template <int CAND>
__global__ __launch_bounds__(64) void route_rows(const float* __restrict__ logits, uint32_t* __restrict__ indices,
                                                 float* __restrict__ weights, uint32_t experts, uint32_t selected,
                                                 uint32_t mode, uint32_t normalize, uint32_t tokens, uint32_t* error_word) {
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    if (row >= tokens) return;
    const float* row_logits = logits + uint64_t(row) * experts;
    uint32_t cand[CAND];
    uint32_t bad = 0;
#pragma unroll
    for (int k = 0; k < CAND; ++k) {
        const uint32_t i = lane + k * kWave;
        uint32_t key = 0;
        if (i < experts) {
            float v = row_logits[i];
            if (nonfinite(v)) { bad |= TSP_ERRBIT_NONFINITE; v = -INFINITY; }
            key = ordered_logit(v);
        }
        cand[k] = key;
    }
    // chosen logit j is kept by lane j (selected <= 64)
    float chosen_mine = 0, chosen_first = 0;
    for (uint32_t s = 0; s < selected; ++s) {
        uint32_t local = 0;
#pragma unroll
        for (int k = 0; k < CAND; ++k) local = cand[k] > local ? cand[k] : local;
        const uint32_t best = wave_extreme_u32<true>(local);
        // the lowest expert id that holds the largest logit: lane + 64 * (first slot of the lane that holds it)
        uint32_t first_slot = CAND;
#pragma unroll
        for (int k = CAND - 1; k >= 0; --k) first_slot = cand[k] == best ? uint32_t(k) : first_slot;
        const bool holds = best != 0 && first_slot < uint32_t(CAND);
        const uint64_t holders = __builtin_amdgcn_ballot_w64(holds);
        uint32_t chosen = 0;
        if (holders == 0) {
            bad |= TSP_ERRBIT_INDEX;
        } else if ((holders & (holders - 1)) == 0) {  // one lane holds it: no tie between lanes to settle
            const int winner = __builtin_ctzll(holders);
            chosen = uint32_t(winner) + kWave * uint32_t(__builtin_amdgcn_readlane(int(first_slot), winner));
        } else {
            chosen = wave_extreme_u32<false>(holds ? lane + kWave * first_slot : 0xffffffffu);
        }
        if (chosen >= experts) { bad |= TSP_ERRBIT_INDEX; chosen = 0; }
        if (lane == 0) indices[uint64_t(row) * selected + s] = chosen;
        const float value = holders == 0 ? row_logits[chosen] : logit_of_ordered(best);
        if (s == 0) chosen_first = value;
        if (s == lane) chosen_mine = value;
        const uint32_t taken = (holders != 0 && chosen % kWave == lane) ? chosen / kWave : uint32_t(CAND);
#pragma unroll
        for (int k = 0; k < CAND; ++k) cand[k] = uint32_t(k) == taken ? 0u : cand[k];
    }
    const float act = lane < selected ? route_activation(chosen_mine, chosen_first, mode, normalize) : 0.0f;
    float sum = mode ? 1.0f : 0.0f;
    if (normalize) {
        sum = wave_sum_shfl(act);
    } else if (!mode) {
        float part = 0;
        for (uint32_t i = lane; i < experts; i += kWave) part += expf(row_logits[i] - chosen_first);
        sum = wave_sum_shfl(part);
    }
    if (nonfinite(sum) || !(sum > 0.0f)) { bad |= TSP_ERRBIT_NONFINITE; sum = 1.0f; }
    if (lane < selected) {
        const float w = act / sum;
        if (nonfinite(w)) bad |= TSP_ERRBIT_NONFINITE;
        weights[uint64_t(row) * selected + lane] = w;
    }
    publish_error(bad, error_word);
}

struct MixtureArgs {
    const float* experts;       // [tokens, selected, channels]
    const float* weights;       // [tokens, selected]
    const float* shared;        // [tokens, channels]
    const float* shared_logit;  // [tokens]
    float* output;
    uint64_t output_stride_bytes;
    uint32_t channels, selected, tokens;
    uint32_t* error_word;
};

__global__ __launch_bounds__(256) void mixture_rows(MixtureArgs a) {
    const uint32_t channel = blockIdx.x * blockDim.x + threadIdx.x, row = blockIdx.y;
    uint32_t bad = 0;
    if (channel < a.channels && row < a.tokens) {
        const float slogit = a.shared_logit[row];
        if (nonfinite(slogit)) {
            bad = TSP_ERRBIT_NONFINITE;
        } else {
            const float* ex = a.experts + uint64_t(row) * a.selected * a.channels + channel;
            const float* w = a.weights + uint64_t(row) * a.selected;
            float value = a.shared[uint64_t(row) * a.channels + channel] * sigmoid_f(slogit);
            for (uint32_t r = 0; r < a.selected; ++r) {
                const float wr = w[r];
                if (nonfinite(wr) || wr < 0.0f) bad = TSP_ERRBIT_NONFINITE;
                value = __builtin_fmaf(wr, ex[uint64_t(r) * a.channels], value);
            }
            if (nonfinite(value)) bad = TSP_ERRBIT_NONFINITE;
            reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(a.output) + row * a.output_stride_bytes)[channel] = value;
        }
    }
    publish_error(bad, a.error_word);
}

// The same with four channels per thread (16-byte loads) and all expert rows of a token requested before the first
// is used; SELECTED = 0 takes the count from the arguments.
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int SELECTED>
__global__ __launch_bounds__(256) void mixture_rows_x4(MixtureArgs a) {
    const uint32_t channel = (blockIdx.x * blockDim.x + threadIdx.x) * 4, row = blockIdx.y;
    const uint32_t selected = SELECTED ? SELECTED : a.selected;
    uint32_t bad = 0;
    if (channel < a.channels && row < a.tokens) {
        const float slogit = a.shared_logit[row];
        if (nonfinite(slogit)) {
            bad = TSP_ERRBIT_NONFINITE;
        } else {
            const float* ex = a.experts + uint64_t(row) * selected * a.channels + channel;
            const float* w = a.weights + uint64_t(row) * selected;
            const f32x4 sh = *reinterpret_cast<const f32x4*>(a.shared + uint64_t(row) * a.channels + channel);
            const float gate = sigmoid_f(slogit);
            f32x4 value = sh * gate;
            auto add = [&](float wr, const f32x4& e) {
                if (nonfinite(wr) || wr < 0.0f) bad = TSP_ERRBIT_NONFINITE;
                value.x = __builtin_fmaf(wr, e.x, value.x); value.y = __builtin_fmaf(wr, e.y, value.y);
                value.z = __builtin_fmaf(wr, e.z, value.z); value.w = __builtin_fmaf(wr, e.w, value.w);
            };
            if constexpr (SELECTED != 0) {
                f32x4 e[SELECTED];
#pragma unroll
                for (int r = 0; r < SELECTED; ++r) e[r] = *reinterpret_cast<const f32x4*>(ex + uint64_t(r) * a.channels);
#pragma unroll
                for (int r = 0; r < SELECTED; ++r) add(w[r], e[r]);
            } else {
                for (uint32_t r = 0; r < selected; ++r) add(w[r], *reinterpret_cast<const f32x4*>(ex + uint64_t(r) * a.channels));
            }
            if (nonfinite(value.x) || nonfinite(value.y) || nonfinite(value.z) || nonfinite(value.w)) bad = TSP_ERRBIT_NONFINITE;
            *reinterpret_cast<f32x4*>(reinterpret_cast<uint8_t*>(a.output) + row * a.output_stride_bytes + uint64_t(channel) * 4) = value;
        }
    }
    publish_error(bad, a.error_word);
}

__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                     float* __restrict__ out, uint64_t count, float scale, uint32_t* error_word) {
    uint32_t bad = 0;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x) {
        const float x = gate[i] * scale, u = up[i];
        float r;
        if (nonfinite(x)) {
            r = x;
            bad = TSP_ERRBIT_NONFINITE;
        } else {
            const float activated = x * sigmoid_f(x);
            if (nonfinite(activated) || nonfinite(u)) { bad = TSP_ERRBIT_NONFINITE; continue; }
            r = activated * u;
            if (nonfinite(r)) bad = TSP_ERRBIT_NONFINITE;
        }
        out[i] = r;
    }
    publish_error(bad, error_word);
}

int route_common(const float* logits, uint32_t* indices, float* weights, uint32_t experts, uint32_t selected, uint32_t tokens,
                 uint32_t mode, int normalize, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(logits && indices && weights && error_word, "null device pointer");
    const uint64_t lb = uint64_t(tokens) * experts * 4, ob = uint64_t(tokens) * selected * 4;
    TSP_REQUIRE(!ranges_overlap(indices, ob, logits, lb) && !ranges_overlap(weights, ob, logits, lb) &&
                    !ranges_overlap(indices, ob, weights, ob),
                "router outputs overlap");
    const auto s = static_cast<hipStream_t>(stream);
    if (experts <= 512) TSP_LAUNCH("route_rows", s, route_rows<8><<<tokens, 64, 0, s>>>(logits, indices, weights, experts, selected, mode, normalize != 0, tokens, error_word));
    else TSP_LAUNCH("route_rows", s, route_rows<64><<<tokens, 64, 0, s>>>(logits, indices, weights, experts, selected, mode, normalize != 0, tokens, error_word));
    return launch_status("route");
}

}  // namespace

extern "C" int tsp_route(const float* logits, uint32_t* indices, float* weights, uint32_t experts, uint32_t selected,
                         uint32_t mode, int normalize_selected, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(experts && experts <= 4096 && selected && selected <= 64 && selected <= experts && mode <= 1,
                "graph router shape/mode mismatch");
    return route_common(logits, indices, weights, experts, selected, 1, mode, normalize_selected, error_word, stream);
}

extern "C" int tsp_route_batch(const float* logits, uint32_t* indices, float* weights, uint32_t experts, uint32_t selected,
                               uint32_t tokens, uint32_t mode, int normalize_selected, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(experts && experts <= 512 && selected && selected <= 64 && selected <= experts && tokens >= 1 && tokens <= 2048 &&
                    mode <= 1,
                "prefill route batch geometry/mode mismatch");
    return route_common(logits, indices, weights, experts, selected, tokens, mode, normalize_selected, error_word, stream);
}

extern "C" int tsp_mixture_batch(const float* experts, const float* weights, const float* shared, const float* shared_logit,
                                 float* output, uint64_t output_stride_bytes, uint32_t channels, uint32_t selected, uint32_t tokens,
                                 uint32_t* error_word, void* stream) {
    TSP_REQUIRE(channels && channels <= 65536 && selected && selected <= 64 && tokens && tokens <= 2048 &&
                    output_stride_bytes >= uint64_t(channels) * 4 && output_stride_bytes % 4 == 0,
                "mixture shape mismatch");
    TSP_REQUIRE(experts && weights && shared && shared_logit && output && error_word, "null device pointer");
    const uint64_t out_span = uint64_t(tokens - 1) * output_stride_bytes + uint64_t(channels) * 4;
    TSP_REQUIRE(!ranges_overlap(output, out_span, experts, uint64_t(tokens) * selected * channels * 4) &&
                    !ranges_overlap(output, out_span, weights, uint64_t(tokens) * selected * 4) &&
                    !ranges_overlap(output, out_span, shared, uint64_t(tokens) * channels * 4) &&
                    !ranges_overlap(output, out_span, shared_logit, uint64_t(tokens) * 4),
                "mixture output overlaps an input");
    const MixtureArgs a{experts, weights, shared, shared_logit, output, output_stride_bytes, channels, selected, tokens, error_word};
    const auto st = static_cast<hipStream_t>(stream);
    const bool wide = channels % 4 == 0 && output_stride_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(experts) | reinterpret_cast<uintptr_t>(shared) |
                                                                            reinterpret_cast<uintptr_t>(output)) % 16 == 0;
    const dim3 grid4((channels / 4 + 255) / 256, tokens);
    if (wide && selected == 10) TSP_LAUNCH("mixture_rows", st, mixture_rows_x4<10><<<grid4, 256, 0, st>>>(a));
    else if (wide && selected == 8) TSP_LAUNCH("mixture_rows", st, mixture_rows_x4<8><<<grid4, 256, 0, st>>>(a));
    else if (wide) TSP_LAUNCH("mixture_rows", st, mixture_rows_x4<0><<<grid4, 256, 0, st>>>(a));
    else TSP_LAUNCH("mixture_rows", st, mixture_rows<<<dim3((channels + 255) / 256, tokens), 256, 0, st>>>(a));
    return launch_status("mixture");
}

extern "C" int tsp_mixture(const float* experts, const float* weights, const float* shared, const float* shared_logit,
                           float* output, uint32_t channels, uint32_t selected, uint32_t* error_word, void* stream) {
    return tsp_mixture_batch(experts, weights, shared, shared_logit, output, uint64_t(channels) * 4, channels, selected, 1,
                             error_word, stream);
}

extern "C" int tsp_swiglu(const float* gate, const float* up, float* output, uint64_t count, float scale, uint32_t* error_word,
                          void* stream) {
    TSP_REQUIRE(count && count <= (1ull << 32) && scale == scale && scale - scale == 0.0f, "graph SwiGLU shape/scale mismatch");
    TSP_REQUIRE(gate && up && output && error_word, "null device pointer");
    TSP_REQUIRE(!ranges_overlap(output, count * 4, up, count * 4) && (output == gate || !ranges_overlap(output, count * 4, gate, count * 4)),
                "SwiGLU output overlaps an input");
    const uint64_t blocks = (count + 255) / 256;
    TSP_LAUNCH("swiglu", static_cast<hipStream_t>(stream), swiglu_kernel<<<uint32_t(blocks > 4096 ? 4096 : blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(gate, up, output, count, scale, error_word));
    return launch_status("swiglu");
}
