// TEST INFRASTRUCTURE ONLY.
//
// extern "C" doorway onto the reference's own CPU functions, compiled together with the reference
// sources where they lie (see build_ref.sh). The resulting library lives in oracle/_ref/ and is
// only ever used to check the C restatement in tokspur_oracle.c and as an optional CPU timing
// baseline. This file contains no arithmetic of its own: every entry converts a FormatError into
// status 1 and forwards.
#include "tokspur/expert_lanes.hpp"
#include "tokspur/gguf.hpp"
#include "tokspur/grouped_mm.hpp"
#include "tokspur/moe_mm_many.hpp"
#include "tokspur/numeric.hpp"
#include "tokspur/operators.hpp"
#include "tokspur/q8_many.hpp"
#include "tokspur/routing.hpp"
#include "tokspur/sampling.hpp"

#include <algorithm>
#include <cstring>

using namespace tokspur;

namespace {
template <class F> int guarded(F&& f) {
    try { f(); return 0; } catch (const FormatError&) { return 1; } catch (...) { return 2; }
}
std::span<const std::byte> bytes(const uint8_t* p, uint64_t n) { return {reinterpret_cast<const std::byte*>(p), size_t(n)}; }
}

extern "C" {

float ref_binary16(uint16_t bits) { return binary16(bits); }

int ref_encoding(uint32_t type, uint32_t* elements, uint32_t* block_bytes) {
    return guarded([&] { const auto& e = encoding(type); *elements = e.elements_per_block; *block_bytes = e.bytes_per_block; });
}

int ref_dequantize(uint32_t type, const uint8_t* data, uint64_t nbytes, float* out, uint64_t nelem) {
    return guarded([&] { dequantize(type, bytes(data, nbytes), std::span<float>(out, size_t(nelem))); });
}

int ref_reference_gemv(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns, uint32_t rows,
                       const float* x, uint64_t nx, double* y) {
    return guarded([&] {
        const auto r = reference_gemv(type, bytes(matrix, nbytes), columns, rows, std::span<const float>(x, size_t(nx)));
        std::copy(r.begin(), r.end(), y);
    });
}

int ref_reference_gemv_doubleinput(uint32_t type, const uint8_t* matrix, uint64_t nbytes, uint32_t columns,
                                   uint32_t rows, const double* x, uint64_t nx, double* y) {
    return guarded([&] {
        const auto r = reference_gemv_doubleinput(type, bytes(matrix, nbytes), columns, rows, std::span<const double>(x, size_t(nx)));
        std::copy(r.begin(), r.end(), y);
    });
}

int ref_reference_q8_many(const uint8_t* matrix, uint64_t nbytes, const float* input, uint32_t columns, uint32_t rows,
                          uint32_t width, double* out) {
    return guarded([&] {
        const auto r = reference_q8_many(bytes(matrix, nbytes), std::span<const float>(input, size_t(columns) * width),
                                         {columns, rows, width}, ~0ull);
        std::copy(r.begin(), r.end(), out);
    });
}
int ref_q8_many_width(uint32_t remaining, uint32_t* width) { return guarded([&] { *width = q8_many_width(remaining); }); }
int ref_q8_many_chunks(uint32_t rows, uint32_t* chunks) { return guarded([&] { *chunks = q8_many_chunks(rows); }); }

int ref_stable_sigmoid(double v, double* out) { return guarded([&] { *out = stable_sigmoid(v); }); }
int ref_stable_silu(double v, double* out) { return guarded([&] { *out = stable_silu(v); }); }
int ref_stable_softplus(double v, double* out) { return guarded([&] { *out = stable_softplus(v); }); }
int ref_group_rms_reference(const double* input, const double* gains, uint64_t count, uint64_t group_width, double epsilon, double* output) {
    return guarded([&] {
        const auto r = group_rms_reference(std::span<const double>(input, size_t(count)), std::span<const double>(gains, size_t(count)), size_t(group_width), epsilon);
        std::copy(r.begin(), r.end(), output);
    });
}
int ref_gated_residual_reference(const double* streams, const double* gains, const double* down, const double* up, const double* inject,
                                 uint64_t branches, uint64_t channels, uint64_t rank, double epsilon, double* read, double* write_scales) {
    return guarded([&] {
        const size_t width = size_t(branches * channels);
        const auto r = gated_residual_reference(std::span<const double>(streams, width), std::span<const double>(gains, width),
                                                std::span<const double>(down, width * size_t(rank)), std::span<const double>(up, width * size_t(rank)),
                                                std::span<const double>(inject, width * size_t(branches)), size_t(branches), size_t(channels), size_t(rank), epsilon);
        std::copy(r.input.begin(), r.input.end(), read);
        std::copy(r.write_scales.begin(), r.write_scales.end(), write_scales);
    });
}
int ref_residual_write_reference(const double* streams, const double* output, const double* scales, uint64_t branches, uint64_t channels, double* result) {
    return guarded([&] {
        const auto r = residual_write_reference(std::span<const double>(streams, size_t(branches * channels)), std::span<const double>(output, size_t(channels)),
                                                std::span<const double>(scales, size_t(branches)));
        std::copy(r.begin(), r.end(), result);
    });
}

int ref_route_reference(const double* logits, uint64_t count, uint64_t selected, uint32_t mode, int normalize,
                        uint32_t* ids, double* weights) {
    return guarded([&] {
        const auto r = route_reference(std::span<const double>(logits, size_t(count)), size_t(selected),
                                       static_cast<RouterMode>(mode), normalize != 0);
        std::copy(r.indices.begin(), r.indices.end(), ids);
        std::copy(r.weights.begin(), r.weights.end(), weights);
    });
}

int ref_mixture_reference(const double* experts, const double* weights, uint64_t nweights, const double* shared,
                          uint64_t channels, double shared_logit, double* out) {
    return guarded([&] {
        const auto r = mixture_reference(std::span<const double>(experts, size_t(nweights * channels)),
                                         std::span<const double>(weights, size_t(nweights)),
                                         std::span<const double>(shared, size_t(channels)), shared_logit);
        std::copy(r.begin(), r.end(), out);
    });
}

int ref_q8_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    return guarded([&] { *offset = lanes::packed_quant_offset(lanes::row_layout(8, columns), block, index); });
}
int ref_q8_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t nbytes) {
    return guarded([&] {
        lanes::pack_rows(lanes::row_layout(8, columns), bytes(original, nbytes),
                         std::span<std::byte>(reinterpret_cast<std::byte*>(packed), size_t(nbytes)));
    });
}
int ref_q8_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t nbytes) {
    return guarded([&] {
        lanes::unpack_rows(lanes::row_layout(8, columns), bytes(packed, nbytes),
                           std::span<std::byte>(reinterpret_cast<std::byte*>(original), size_t(nbytes)));
    });
}

int ref_q51_lanes_quant_offset(uint32_t columns, uint32_t block, uint32_t index, uint64_t* offset) {
    return guarded([&] { *offset = lanes::packed_quant_offset(lanes::row_layout(7, columns), block, index); });
}
int ref_q51_lanes_pack_rows(uint32_t columns, const uint8_t* original, uint8_t* packed, uint64_t nbytes) {
    return guarded([&] {
        lanes::pack_rows(lanes::row_layout(7, columns), bytes(original, nbytes),
                         std::span<std::byte>(reinterpret_cast<std::byte*>(packed), size_t(nbytes)));
    });
}
int ref_q51_lanes_unpack_rows(uint32_t columns, const uint8_t* packed, uint8_t* original, uint64_t nbytes) {
    return guarded([&] {
        lanes::unpack_rows(lanes::row_layout(7, columns), bytes(packed, nbytes),
                           std::span<std::byte>(reinterpret_cast<std::byte*>(original), size_t(nbytes)));
    });
}

int ref_logit_topk_row(const float* logits, uint64_t n, void* out528) {
    return guarded([&] {
        const auto row = cpu_logit_topk_row(std::span<const float>(logits, size_t(n)));
        static_assert(sizeof(row) == 528);
        std::memcpy(out528, &row, sizeof row);
    });
}

// Fills the same 104-byte record tokspur_oracle.h declares as orc_grouped_mm_plan.
int ref_grouped_mm_plan(uint32_t type, uint32_t layout, uint32_t columns, uint32_t rows, uint32_t experts,
                        uint32_t selected, uint32_t tokens, uint64_t input_stride, uint64_t output_stride,
                        int broadcast, int allow_nax_2k, void* out) {
    return guarded([&] {
        const auto p = grouped_mm_plan(type, static_cast<PrefillWeightLayout>(layout), columns, rows, experts, selected,
                                       tokens, input_stride, output_stride, broadcast != 0, allow_nax_2k != 0);
        auto* dst = static_cast<uint8_t*>(out);
        std::memcpy(dst, &p.args, 56);
        const uint64_t spans[7] = {p.matrix_bytes, p.indices_bytes, p.input_bytes, p.output_bytes,
                                   p.token_map_bytes, p.counts_bytes, p.tasks_bytes};
        std::memcpy(dst + 56, spans, 56);
        const uint32_t grid[2] = {p.grid_x, p.grid_y};
        std::memcpy(dst + 112, grid, 8);
    });
}

int ref_moe_mm_many_bytes(uint32_t channels, uint32_t hidden, uint32_t experts, uint32_t selected, uint32_t capacity,
                          int allow_nax_2k, uint64_t* views13, uint64_t* total) {
    return guarded([&] {
        const auto b = moe_mm_many_bytes({channels, hidden, experts, selected}, capacity, allow_nax_2k != 0);
        std::copy(b.views.begin(), b.views.end(), views13);
        *total = b.total;
    });
}

}
