// Grouped dequant-GEMM with weights and activations staged as halves (see grouped_staged.hip).
#pragma once

#include "tsp_common.hpp"

namespace tsp {

struct GroupedStagedArgs {
    const uint8_t* matrices;   // [experts][rows][row_bytes]
    const float* input;        // f32 rows, one per token (broadcast) or per route
    float* output;             // f32 rows, one per route
    uint64_t expert_stride, input_stride, output_stride;  // bytes
    uint32_t columns, rows, row_bytes, experts, selected, tokens, broadcast, maximum_tasks;
    const uint32_t* ids;
    const uint32_t* token_map;
    const uint32_t* counts;
    const uint32_t* tasks;     // the engine's list of 32-route tasks: [count, routes, (expert, start) ...]
    uint32_t* error_word;
};

bool grouped_staged_takes(uint32_t encoding, uint32_t layout);
int launch_grouped_staged(uint32_t encoding, uint32_t layout, const GroupedStagedArgs& args, hipStream_t stream);

}  // namespace tsp
