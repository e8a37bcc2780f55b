// ragged u16 index lists (per-task entry counts) whose fields are row*4.
#include "lists.hpp"

namespace sptmm {

int launch_ragged_u16_scaled(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<0, true, true>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
