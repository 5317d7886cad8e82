// Instantiates the MFMA split-KV decode kernels for one KV-cache element kind (f16).
#include "decode_mfma_kernels.hpp"

namespace areno {
decode_mfma_fn decode_mfma_lookup_f16(int head_dim, bool scale16) {
  return decode_mfma_lookup_impl<KV_F16>(head_dim, scale16);
}
}  // namespace areno
