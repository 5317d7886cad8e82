// Instantiates the MFMA split-KV decode kernels for one KV-cache element kind (fp8): the plain kernel and the one
// that reads shared prefix pages once per group of rows.
#include "decode_mfma_kernels.hpp"

namespace areno {
decode_mfma_fn decode_mfma_lookup_fp8(int head_dim, bool scale16, bool grouped) {
  return grouped ? decode_mfma_lookup_impl<KV_FP8, true>(head_dim, scale16)
                 : decode_mfma_lookup_impl<KV_FP8, false>(head_dim, scale16);
}
}  // namespace areno
