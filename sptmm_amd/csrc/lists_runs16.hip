// run gap stream, 16-bit gaps.
#include "lists.hpp"

namespace sptmm {

int launch_runs16(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<2, false, false>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
