// Instantiates the split-KV decode kernels for one KV-cache element kind (f16); one unit per kind so
// the units compile in parallel.
#include "paged_decode_kernels.hpp"

namespace areno {
decode_split_fn decode_split_lookup_f16(int head_dim, int group) {
  return decode_split_lookup_impl<KV_F16>(head_dim, group);
}
}  // namespace areno
