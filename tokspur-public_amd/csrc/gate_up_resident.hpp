// Launch interface of the activation-resident grouped gate/up kernel (gate_up_resident.hip).
#pragma once
#include "tsp_common.hpp"

namespace tsp {

struct ResidentGateUpArgs {
    const _Float16* xh;       // [tokens][2048] activations as halves, columns 1 <-> 2 and 5 <-> 6 of every eight swapped
    const _Float16* sx;       // [tokens][8][16] sub-block sums of those rows: eight high halves, eight residuals
    const uint8_t* pair_lo;   // co-located [gate_e, up_e] Pack v3 Q4_K experts 0 .. experts/2-1
    const uint8_t* pair_hi;   // the same for experts/2 .. experts-1
    const uint8_t* shared_gate;  // an always-on expert whose tasks carry expert id == experts (null: none)
    const uint8_t* shared_up;
    tsp_planar_spec spec;     // one expert: 2048 columns, `hidden` rows
    uint32_t experts, tokens, selected, hidden;
    const uint32_t* tasks;    // [2 + 2 * task_slots]: live tasks, routes, then (expert, first row) per 64-row task
    const uint32_t* classes;  // [2 + 2 * task_slots]: tasks of <= 32 rows, tasks of 33..64 rows, then the two kinds' task indices
    const uint32_t* counts;
    const uint32_t* token_map;
    const uint32_t* ids;
    uint32_t task_slots;
    _Float16* hbuf;           // [task_slots * 64][hidden]: SwiGLU output rows by task slot, as halves of h / 256
    uint32_t* error_word;
};

bool resident_gate_up_takes(uint32_t channels, uint32_t hidden);
int launch_resident_gate_up(const ResidentGateUpArgs& args, hipStream_t stream);

}  // namespace tsp
