// ragged u16 index lists (per-task entry counts) whose fields are plain row indices.
#include "lists.hpp"

namespace sptmm {

int launch_ragged_u16_plain(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<0, false, true>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
