// u16 index lists whose fields are row*4 (4K fits 16 bits).
#include "lists.hpp"

namespace sptmm {

int launch_u16_scaled(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<0, true, false>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
