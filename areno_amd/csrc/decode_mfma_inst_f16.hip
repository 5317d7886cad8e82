// Instantiates the MFMA split-KV decode kernels for one KV-cache element kind (f16): the plain kernel and the one
// that reads shared prefix pages once per group of rows.
#include "decode_mfma_kernels.hpp"

namespace areno {
decode_mfma_fn decode_mfma_lookup_f16(int head_dim, bool scale16, bool grouped) {
  return grouped ? decode_mfma_lookup_impl<KV_F16, true>(head_dim, scale16)
                 : decode_mfma_lookup_impl<KV_F16, false>(head_dim, scale16);
}
}  // namespace areno
