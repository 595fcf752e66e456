// The small f32 operators that sit either side of the MoE sublayer in a layer (kernels/graph.metal:222-361): grouped RMS
// normalisation (alone and fused with a sigmoid gate), activations, gated multiplication, and the read / write of the gated
// residual streams. All are a few bytes per element and bound by memory or by launch latency; they follow the engine's error
// contract: a non-finite result sets the sticky bit and is stored all the same (kernels/graph.metal:18-21), so after a refused
// batch a destination holds what the engine's holds; a non-finite INPUT of the operators that test their inputs first
// (multiply, the gated RMS, residual_read) sets the bit and leaves that element of the destination as it was.
#include "tsp_common.hpp"

using namespace tsp;

namespace {

// kernels/graph.metal:4-16
__device__ __forceinline__ float sigmoid_value(float x) {
    if (x >= 0) return 1.0f / (1.0f + expf(-x));
    const float e = expf(x);
    return e / (1.0f + e);
}
__device__ __forceinline__ float softplus_value(float x) {
    const float z = expf(-fabsf(x)), sum = 1.0f + z;
    // log1p by compensation: 1 + z rounds, (sum - 1) is what was actually added; a sum that rounds to 1 keeps its tiny tail
    return fmaxf(x, 0.0f) + (sum == 1.0f ? z : logf(sum) * (z / (sum - 1.0f)));
}
// kernels/graph.metal:18-21: the value is stored whatever it is; a non-finite one raises the flag as well
__device__ __forceinline__ uint32_t checked_store(float* out, uint64_t i, float v) {
    out[i] = v;
    return nonfinite(v) ? TSP_ERRBIT_NONFINITE : 0u;
}

// One wave per group of `width` values: out = x * rsqrt(mean(x^2) + eps) * gain, gains per element or shared by all groups;
// GATED multiplies by sigmoid(gate) as well.
template <bool GATED>
__global__ __launch_bounds__(256) void rms_kernel(const float* __restrict__ input, const float* __restrict__ gains, const float* __restrict__ gate,
                                                  float* __restrict__ output, uint32_t groups, uint32_t width, uint32_t shared_gains, float epsilon,
                                                  uint32_t* error_word) {
    const uint32_t lane = threadIdx.x % kWave, group = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (group >= groups) return;
    const uint64_t base = uint64_t(group) * width;
    float squared = 0;
    for (uint32_t i = lane; i < width; i += kWave) squared += input[base + i] * input[base + i];
    const float total = wave_sum(squared), denominator = total / float(width) + epsilon;
    uint32_t bad = 0;
    if (nonfinite(total) || nonfinite(denominator)) {
        bad = TSP_ERRBIT_NONFINITE;
    } else {
        const float inverse = 1.0f / sqrtf(denominator);
        for (uint32_t i = lane; i < width; i += kWave) {
            const float normalised = input[base + i] * inverse * gains[(shared_gains ? 0 : base) + i];
            if constexpr (GATED) {
                const float g = gate[base + i];
                if (nonfinite(normalised) || nonfinite(g)) { bad = TSP_ERRBIT_NONFINITE; continue; }
                bad |= checked_store(output, base + i, normalised * sigmoid_value(g));
            } else {
                bad |= checked_store(output, base + i, normalised);
            }
        }
    }
    publish_error(bad, error_word);
}

__global__ __launch_bounds__(256) void activate_kernel(const float* input, float* output, uint64_t count, uint32_t kind, float scale, uint32_t* error_word) {
    uint32_t bad = 0;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x) {
        const float x = input[i] * scale;
        float value = x;  // a bounded activation must not hide a non-finite input: it is refused before it is mapped
        if (!nonfinite(x)) value = kind == 1 ? x * sigmoid_value(x) : kind == 2 ? sigmoid_value(x) : kind == 3 ? softplus_value(x) : x;
        bad |= checked_store(output, i, value);
    }
    publish_error(bad, error_word);
}

__global__ __launch_bounds__(256) void multiply_kernel(const float* input, const float* gate, float* output, uint64_t count, uint32_t sigmoid_gate,
                                                       uint32_t* error_word) {
    uint32_t bad = 0;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x) {
        const float x = input[i], g = gate[i];
        if (nonfinite(x) || nonfinite(g)) { bad = TSP_ERRBIT_NONFINITE; continue; }
        bad |= checked_store(output, i, x * (sigmoid_gate ? sigmoid_value(g) : g));
    }
    publish_error(bad, error_word);
}

// output[c] = mean over branches of normalised[b, c] * sigmoid(scores[b, c]); scales[b] = 2 sigmoid(inject[b] / branches)
__global__ __launch_bounds__(256) void residual_read_kernel(const float* __restrict__ normalised, const float* __restrict__ scores,
                                                            const float* __restrict__ inject, float* __restrict__ output, float* __restrict__ scales,
                                                            uint32_t branches, uint32_t channels, uint32_t* error_word) {
    const uint32_t channel = blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t bad = 0;
    bool ok = true;  // a thread that met a non-finite operand writes nothing more, neither its channel nor its scale (graph.metal:340)
    if (channel < channels) {
        float total = 0;
        for (uint32_t b = 0; b < branches && ok; ++b) {
            const float n = normalised[uint64_t(b) * channels + channel], s = scores[uint64_t(b) * channels + channel];
            if (nonfinite(n) || nonfinite(s)) { bad = TSP_ERRBIT_NONFINITE; ok = false; break; }
            total += n * sigmoid_value(s);
        }
        if (ok) bad |= checked_store(output, channel, total / float(branches));
    }
    if (ok && channel < branches) {
        const float v = inject[channel];
        if (nonfinite(v)) bad = TSP_ERRBIT_NONFINITE;
        else bad |= checked_store(scales, channel, 2.0f * sigmoid_value(v / float(branches)));
    }
    publish_error(bad, error_word);
}

// output[b, c] = streams[b, c] + scales[b] * input[c]
__global__ __launch_bounds__(256) void residual_write_kernel(const float* streams, const float* __restrict__ input, const float* __restrict__ scales,
                                                             float* output, uint32_t branches, uint32_t channels, uint32_t* error_word) {
    const uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x;
    uint32_t bad = 0;
    if (i < uint64_t(branches) * channels) bad = checked_store(output, i, streams[i] + scales[i / channels] * input[i % channels]);
    publish_error(bad, error_word);
}

uint32_t blocks_for(uint64_t count) {
    const uint64_t want = (count + 255) / 256;
    return uint32_t(want < 1 ? 1 : want > 8192 ? 8192 : want);
}

int rms_common(const float* input, const float* gains, const float* gate, float* output, uint64_t count, uint32_t group_width, int shared_gains,
               float epsilon, uint32_t* error_word, void* stream, const char* refusal) {
    TSP_REQUIRE(group_width && group_width <= 65536 && count && count <= (1ull << 32) - 1 && count % group_width == 0 && epsilon == epsilon &&
                    epsilon - epsilon == 0.0f && epsilon > 0,
                "%s", refusal);
    TSP_REQUIRE(input && gains && output && error_word, "null device pointer");
    const uint64_t bytes = count * 4, gain_bytes = (shared_gains ? uint64_t(group_width) : count) * 4;
    TSP_REQUIRE(!ranges_overlap(output, bytes, input, bytes) && !ranges_overlap(output, bytes, gains, gain_bytes) &&
                    !(gate && ranges_overlap(output, bytes, gate, bytes)),
                "RMS output overlaps an input");
    const uint32_t groups = uint32_t(count / group_width);
    const auto s = static_cast<hipStream_t>(stream);
    if (gate) TSP_LAUNCH("rms_sigmoid_gate", s, rms_kernel<true><<<(groups + 3) / 4, 256, 0, s>>>(input, gains, gate, output, groups, group_width, shared_gains != 0, epsilon, error_word));
    else TSP_LAUNCH("rms", s, rms_kernel<false><<<(groups + 3) / 4, 256, 0, s>>>(input, gains, nullptr, output, groups, group_width, shared_gains != 0, epsilon, error_word));
    return launch_status("rms");
}

}  // namespace

extern "C" int tsp_rms(const float* input, const float* gains, float* output, uint64_t count, uint32_t group_width, int shared_gains, float epsilon,
                       uint32_t* error_word, void* stream) {
    return rms_common(input, gains, nullptr, output, count, group_width, shared_gains, epsilon, error_word, stream, "graph RMS shape/epsilon mismatch");
}

extern "C" int tsp_rms_sigmoid_gate(const float* input, const float* gains, const float* gate, float* output, uint64_t count, uint32_t group_width,
                                    int shared_gains, float epsilon, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(gate, "null device pointer");
    return rms_common(input, gains, gate, output, count, group_width, shared_gains, epsilon, error_word, stream, "graph RMS sigmoid gate shape/epsilon mismatch");
}

extern "C" int tsp_activate(const float* input, float* output, uint64_t count, uint32_t kind, float scale, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(count && count <= (1ull << 32) - 1 && kind <= 3 && scale == scale && scale - scale == 0.0f, "graph activation shape/mode mismatch");
    TSP_REQUIRE(input && output && error_word, "null device pointer");
    TSP_REQUIRE(output == input || !ranges_overlap(output, count * 4, input, count * 4), "activation output overlaps its input");  // in place is allowed
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("activate", s, activate_kernel<<<blocks_for(count), 256, 0, s>>>(input, output, count, kind, scale, error_word));
    return launch_status("activate");
}

extern "C" int tsp_multiply(const float* input, const float* gate, float* output, uint64_t count, int sigmoid_gate, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(count && count <= (1ull << 32) - 1, "graph multiplication shape mismatch");
    TSP_REQUIRE(input && gate && output && error_word, "null device pointer");
    TSP_REQUIRE((output == input || !ranges_overlap(output, count * 4, input, count * 4)) && (output == gate || !ranges_overlap(output, count * 4, gate, count * 4)),
                "multiplication output overlaps an input");  // exactly in place is allowed
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("multiply", s, multiply_kernel<<<blocks_for(count), 256, 0, s>>>(input, gate, output, count, sigmoid_gate != 0, error_word));
    return launch_status("multiply");
}

extern "C" int tsp_residual_read(const float* normalized, const float* scores, const float* inject, float* output, float* scales, uint32_t branches,
                                 uint32_t channels, uint32_t* error_word, void* stream) {
    TSP_REQUIRE(branches && branches <= 64 && channels && channels <= 65536, "graph residual-read shape mismatch");
    TSP_REQUIRE(normalized && scores && inject && output && scales && error_word, "null device pointer");
    const uint64_t wide = uint64_t(branches) * channels * 4;
    const void* ins[] = {normalized, scores, inject};
    const uint64_t in_bytes[] = {wide, wide, uint64_t(branches) * 4};
    for (int i = 0; i < 3; ++i)
        TSP_REQUIRE(!ranges_overlap(output, uint64_t(channels) * 4, ins[i], in_bytes[i]) && !ranges_overlap(scales, uint64_t(branches) * 4, ins[i], in_bytes[i]),
                    "residual-read output overlaps an input");
    TSP_REQUIRE(!ranges_overlap(output, uint64_t(channels) * 4, scales, uint64_t(branches) * 4), "residual-read outputs overlap each other");
    const uint32_t threads = branches > channels ? branches : channels;
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("residual_read", s, residual_read_kernel<<<(threads + 255) / 256, 256, 0, s>>>(normalized, scores, inject, output, scales, branches, channels, error_word));
    return launch_status("residual_read");
}

extern "C" int tsp_residual_write(const float* streams, const float* input, const float* scales, float* output, uint32_t branches, uint32_t channels,
                                  uint32_t* error_word, void* stream) {
    TSP_REQUIRE(branches && branches <= 64 && channels && channels <= 65536, "graph residual-write shape mismatch");
    TSP_REQUIRE(streams && input && scales && output && error_word, "null device pointer");
    const uint64_t wide = uint64_t(branches) * channels * 4;
    TSP_REQUIRE(!ranges_overlap(output, wide, input, uint64_t(channels) * 4) && !ranges_overlap(output, wide, scales, uint64_t(branches) * 4) &&
                    (output == streams || !ranges_overlap(output, wide, streams, wide)),
                "residual-write output overlaps an input");  // the streams may be updated in place
    const auto s = static_cast<hipStream_t>(stream);
    TSP_LAUNCH("residual_write", s, residual_write_kernel<<<uint32_t((uint64_t(branches) * channels + 255) / 256), 256, 0, s>>>(streams, input, scales, output, branches, channels, error_word));
    return launch_status("residual_write");
}
