// Launch interface of the h-resident grouped down kernel (down_resident.hip).
#pragma once
#include "tsp_common.hpp"

namespace tsp {

struct ResidentDownArgs {
    const _Float16* hbuf;        // [task_slots * 64][512]: SwiGLU output rows by task slot, as halves of h / 256
    const uint8_t* down;         // Q6_K planes (ql / qh / sub-scales / d), Q8_0 planes (quants / d) or Q5_1 planes (nibbles / fifth bits / d, m) per expert, `channels` rows of 512 columns
    const uint8_t* shared_down;  // an always-on expert whose tasks carry expert id == experts (null: none)
    tsp_planar_spec spec;        // one expert
    uint32_t experts, tokens, selected, channels;
    const uint32_t* tasks;       // [2 + 2 * task_slots]: live tasks, routes, then (expert, first row) per 64-row task
    const uint32_t* classes;     // [2 + 2 * task_slots]: tasks of <= 32 rows, tasks of 33..64 rows, then the two kinds' task indices
    const uint32_t* counts;
    const uint32_t* token_map;
    const uint32_t* ids;
    uint32_t task_slots;
    float* y;                    // [tokens * selected] rows by route, y_stride bytes apart; the whole output spans less than 4 GiB
    uint64_t y_stride;
    float* shared_y;             // the always-on expert's rows by token
    uint64_t shared_y_stride;
    float out_scale;             // 256: undoes the 2^-8 that h carries (a power of two)
    uint32_t* error_word;
};

bool resident_down_takes(uint32_t source_type, uint32_t channels, uint32_t hidden);  // source_type: 14 (Q6_K planes), 8 (Q8_0 planes) or 7 (Q5_1 planes)
int launch_resident_down(const ResidentDownArgs& args, hipStream_t stream);

}  // namespace tsp
