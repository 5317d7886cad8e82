// MFMA (matrix-core) causal prefill over paged KV for gfx950.
#include "device_common.hpp"

namespace areno {

int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* stream) {
  (void)cache; (void)q; (void)out; (void)q_dtype; (void)tokens; (void)q_heads; (void)num_seqs; (void)block_table;
  (void)max_blocks; (void)cu_seqlens_q; (void)context_lens; (void)window_left; (void)softmax_scale; (void)stream;
  return ARENO_ERR_UNSUPPORTED;
}

}  // namespace areno
