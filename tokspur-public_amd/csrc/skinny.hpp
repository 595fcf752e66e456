// Internal interface of the small-row matrix-core kernels (skinny.hip), used by the T <= 8 routed MoE entry points.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

struct SkinnyMoe {
    const uint8_t* pair_lo;  // experts 0..E/2-1 as [gate_e, up_e]
    const uint8_t* pair_hi;  // experts E/2..E-1
    const uint8_t* down;     // [experts] planar
    const uint32_t* ids;     // [tokens * selected]
    uint32_t* meta;          // union records (the caller's scratch: the record-resident launch writes them), or nullptr for one route per task
    const float* x;          // token rows
    float* h;                // route rows
    float* y;                // route rows
    uint64_t x_stride, h_stride, y_stride;  // bytes
    uint32_t channels, hidden, experts, selected, tokens, records;
    tsp_planar_spec gu, dn;
    uint32_t* error_word;
    // optional always-on expert riding in the same launches (one Pack v3 expert each; rows = the tokens)
    const uint8_t* shared_gate = nullptr;
    const uint8_t* shared_up = nullptr;
    const uint8_t* shared_down = nullptr;
    float* shared_h = nullptr;  // [tokens, hidden]
    float* shared_y = nullptr;  // [tokens, channels]
    uint64_t shared_h_stride = 0, shared_y_stride = 0;
};

// Q4_K co-located gate/up (and Q6_K planar down when with_down), columns a multiple of 256 up to 2048, 16-byte aligned rows.
bool skinny_moe_supported(uint32_t gate_up_type, uint32_t down_type, uint32_t channels, uint32_t hidden, const void* x, uint64_t x_stride,
                          const void* h, uint64_t h_stride, bool with_down);
int skinny_moe_gate_up(const SkinnyMoe& m, hipStream_t stream);
int skinny_moe_down(const SkinnyMoe& m, hipStream_t stream);

}  // namespace tsp
