// Arguments shared by the backward kernels of the causal varlen / dense attention ops (attention_backward.hip: the
// vector-ALU kernels for every head dim and dtype; attention_backward_mfma.hip: matrix-core kernels for 16-bit
// inputs at head dims 64 and 128).
#pragma once

#include <stdint.h>

#include "areno_hip.h"

namespace areno {

struct BwdParams {
  const void* grad_out;
  const void* q;
  const void* k;
  const void* v;
  const void* out;
  void* grad_q;  // gradients in fp32, or in the inputs' 16-bit type (grad_dtype)
  void* grad_k;
  void* grad_v;
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
  int32_t grad_dtype;  // ARENO_DT_F32, or `dtype` when that is a 16-bit type: the fp32 sums rounded once, at the store
  float scale;
  float scale_log2e;
};

#if defined(__HIPCC__)
// one gradient element, and four consecutive ones (`i` a multiple of 4), in the type `grad_dtype` names
__device__ inline __attribute__((always_inline)) void store_grad(void* base, int64_t i, float x, int32_t grad_dtype) {
  if (grad_dtype == ARENO_DT_F32) {
    static_cast<float*>(base)[i] = x;
  } else if (grad_dtype == ARENO_DT_BF16) {
    static_cast<__bf16*>(base)[i] = static_cast<__bf16>(x);
  } else {
    static_cast<_Float16*>(base)[i] = static_cast<_Float16>(x);
  }
}
__device__ inline __attribute__((always_inline)) void store_grad4(void* base, int64_t i, float a, float b, float c, float d, int32_t grad_dtype) {
  typedef __attribute__((ext_vector_type(4))) float f32x4;
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
  const f32x4 v = {a, b, c, d};
  if (grad_dtype == ARENO_DT_F32) {
    *reinterpret_cast<f32x4*>(static_cast<float*>(base) + i) = v;
  } else if (grad_dtype == ARENO_DT_BF16) {
    *reinterpret_cast<bf16x4*>(static_cast<__bf16*>(base) + i) = __builtin_convertvector(v, bf16x4);
  } else {
    *reinterpret_cast<f16x4*>(static_cast<_Float16*>(base) + i) = __builtin_convertvector(v, f16x4);
  }
}
#endif

// Matrix-core backward (attention_backward_mfma.hip): launches both kernels on `stream` and returns ARENO_OK, or
// ARENO_ERR_UNSUPPORTED when the shape is not one it serves (the caller then takes the vector-ALU kernels).
int launch_attention_backward_mfma(const BwdParams& p, void* stream);

}  // namespace areno
