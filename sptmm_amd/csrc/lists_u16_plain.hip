// u16 index lists with plain row fields (K above 16383).
#include "lists.hpp"

namespace sptmm {

int launch_u16_plain(const GemvArgs &a, ActType act, void *stream) { return launch_lists_a<0, false>(a, act, (hipStream_t)stream); }

}  // namespace sptmm
