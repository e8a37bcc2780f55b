// gap stream striped by row mod 32, 8-bit gaps of 32 rows.
#include "lists.hpp"

namespace sptmm {

int launch_striped(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<3, false>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
