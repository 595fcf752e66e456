// Internal interface of the activation-resident gate/up + SwiGLU kernel for the T <= 8 routed MoE (record_resident.hip): the
// union records' product for 2048-column Q4_K experts as persistent workgroups that stream the experts' planes through LDS.
#pragma once
#include "skinny.hpp"

namespace tsp {

// Union records present (more than one token), Q4_K gate/up planes of 2048 columns, whole 32-unit tiles, token rows and a
// union block that 16 bytes align.
bool record_gate_up_takes(const SkinnyMoe& m);
int launch_record_gate_up(const SkinnyMoe& m, hipStream_t stream);

}  // namespace tsp
