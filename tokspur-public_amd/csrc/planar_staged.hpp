// Grouped MoE products for the planar kinds decoded to halves on the fly (see planar_staged.hip).
#pragma once

#include "tsp_common.hpp"

namespace tsp {

struct PlanarStagedArgs {
    const _Float16* xh;            // [tokens][channels] activation rows as halves, columns in their natural order
    const uint8_t* pair_lo;        // co-located gate / up halves
    const uint8_t* pair_hi;
    const uint8_t* down;           // [experts] planar down experts
    tsp_planar_spec spec;          // one gate (or up) expert
    tsp_planar_spec down_spec;     // one down expert
    uint32_t channels, hidden, experts, selected, tokens;
    const uint32_t* task_list;     // 64-row tasks: [count, routes, (expert, start) ...]
    uint32_t task_slots;
    const uint32_t* counts;
    const uint32_t* token_map;
    const uint32_t* ids;
    _Float16* hbuf;                // [task slot * 64 + row][hidden]: the half nearest h / 256
    float* y;                      // [route][channels], rows y_stride bytes apart
    uint64_t y_stride;
    uint32_t* error_word;
};

bool planar_staged_gate_up_takes(uint32_t gate_kind, uint32_t up_kind);
bool planar_staged_down_takes(uint32_t down_kind);
int launch_planar_staged_gate_up(const PlanarStagedArgs& args, hipStream_t stream);
int launch_planar_staged_down(const PlanarStagedArgs& args, hipStream_t stream);

}  // namespace tsp
