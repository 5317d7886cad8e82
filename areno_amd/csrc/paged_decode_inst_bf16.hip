// Instantiates the split-KV decode kernels for one KV-cache element kind (bf16); one unit per kind so
// the units compile in parallel.
#include "paged_decode_kernels.hpp"

namespace areno {
decode_split_fn decode_split_lookup_bf16(int head_dim, int group) {
  return decode_split_lookup_impl<KV_BF16>(head_dim, group);
}
}  // namespace areno
