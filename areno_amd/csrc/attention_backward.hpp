// Arguments shared by the backward kernels of the causal varlen / dense attention ops (attention_backward.hip: the
// vector-ALU kernels for every head dim and dtype; attention_backward_mfma.hip: matrix-core kernels for 16-bit
// inputs at head dims 64 and 128).
#pragma once

#include <stdint.h>

namespace areno {

struct BwdParams {
  const void* grad_out;
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  float* grad_q;
  float* grad_k;
  float* grad_v;
  float* row_stats;  // [q_tokens * q_heads][2]: log2-domain log-sum-exp of the scaled scores, dO . O
  const int32_t* cu_q;
  const int32_t* cu_k;
  const int32_t* ctx;  // may be nullptr: 0
  int64_t q_tokens;
  int64_t k_tokens;
  int32_t num_seqs;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t window_left;
  int32_t head_dim;
  int32_t dtype;
  float scale;
  float scale_log2e;
};

// Matrix-core backward (attention_backward_mfma.hip): launches both kernels on `stream` and returns ARENO_OK, or
// ARENO_ERR_UNSUPPORTED when the shape is not one it serves (the caller then takes the vector-ALU kernels).
int launch_attention_backward_mfma(const BwdParams& p, void* stream);

}  // namespace areno
