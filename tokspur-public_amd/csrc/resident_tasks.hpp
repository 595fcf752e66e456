// Shared by the two resident grouped GEMMs (gate_up_resident.hip, down_resident.hip): how a persistent workgroup learns about
// the tasks of its share. A task is an entry of the grouped GEMMs' 64-row task list, (expert, first row); the always-on
// expert's tasks carry expert id == experts and take the tokens themselves as their rows.
#pragma once
#include "tsp_common.hpp"

namespace tsp {

constexpr uint32_t kResidentTaskRows = 64;
constexpr uint32_t kResidentInfoSlots = 32;  // tasks of a workgroup's share kept in LDS, per pass

struct ResidentTask { uint32_t task, expert, start, nrows; bool shared, ok; };

// (task, expert, first row, rows | shared << 8 | ok << 9): one 16-byte LDS slot per task
__device__ __forceinline__ uint4 pack_resident_task(const ResidentTask& t) {
    return uint4{t.task, t.expert, t.start, t.nrows | (t.shared ? 256u : 0u) | (t.ok ? 512u : 0u)};
}
// The words are the same in every lane (every lane read the same slot): they go to scalar registers.
__device__ __forceinline__ ResidentTask unpack_resident_task(const uint4& v) {
    ResidentTask t;
    t.task = __builtin_amdgcn_readfirstlane(v.x);
    t.expert = __builtin_amdgcn_readfirstlane(v.y);
    t.start = __builtin_amdgcn_readfirstlane(v.z);
    const uint32_t w = __builtin_amdgcn_readfirstlane(v.w);
    t.nrows = w & 255u; t.shared = (w & 256u) != 0; t.ok = (w & 512u) != 0;
    return t;
}

// The task at list entry `listed_task` of a launch with `listed` tasks. A task that does not check out (expert out of range,
// more rows than tokens, first row past the expert's count) keeps addresses inside the tensors (expert 0, row 0) and has no
// rows; whoever resolves it flags the batch.
__device__ __forceinline__ ResidentTask resolve_resident_task(const uint32_t* __restrict__ tasks, const uint32_t* __restrict__ counts,
                                                              uint32_t listed_task, uint32_t listed, uint32_t experts, uint32_t tokens,
                                                              bool has_shared) {
    ResidentTask t;
    t.task = listed_task < listed ? listed_task : 0;
    t.expert = tasks[2 + 2 * t.task];
    t.start = tasks[3 + 2 * t.task];
    t.shared = has_shared && t.expert == experts;
    const uint32_t count = t.shared ? tokens : t.expert < experts ? counts[t.expert] : 0;
    t.ok = (t.expert < experts || t.shared) && count <= tokens && t.start < count;
    t.nrows = t.ok ? (count - t.start < kResidentTaskRows ? count - t.start : kResidentTaskRows) : 0;
    if (!t.ok) { t.expert = 0; t.start = 0; t.shared = false; }
    return t;
}

}  // namespace tsp
