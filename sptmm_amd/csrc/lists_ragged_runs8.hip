// ragged run gap stream (per-task entry counts), 8-bit gaps.
#include "lists.hpp"

namespace sptmm {

int launch_ragged_runs8(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<1, false, true>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
