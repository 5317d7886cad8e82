// Backward of the causal varlen / dense attention ops (gfx950): dQ, dK, dV in fp32 from dO, Q, K, V and the saved
// output, the contract of the reference's backward kernels (areno/accel/csrc/attention.cu:244-524: one thread block
// per (token, head) row, three passes over the row's keys, atomicAdd into dK / dV).  This is the training-side
// companion of the inference path, written for correctness and determinism, not for the matrix cores:
//
//   rows kernel   one wave per (query token, q head): 16 keys at a time, 4 lanes per key (each lane owns a quarter of
//                 the head dimension), pass 1 for the row's softmax statistics, pass 2 for
//                   dS_j = P_j * (dO . V_j - dO . O)   and   dQ += scale * dS_j * K_j
//                 (dO . (V_j - O) in the reference, l.486-497); leaves log-sum-exp and dO . O per row in the workspace
//   keys kernel   one wave per (key token, kv head): 16 (query, head-of-group) pairs at a time, recomputes P and dS
//                 from the saved statistics and accumulates dV_j = sum P dO, dK_j = scale * sum dS Q in registers --
//                 every gradient element has one owner, so there are no atomics and the result does not depend on
//                 scheduling (the reference's atomicAdd order does).
//
// Geometry: sequence s has queries [cu_q[s], cu_q[s+1]) at positions ctx[s] + i and keys [cu_k[s], cu_k[s+1]) at
// positions 0 ..; query at position t sees keys max(0, t - window) .. t.  The varlen op has cu_k = cu_q, ctx = 0; the
// dense op one sequence per batch row with ctx = query_start.
// Head dims that are multiples of 8 up to 256: a lane owns a quarter of the head in registers, 16 / 32 / 48 / 64
// elements wide (the smallest that covers the head; slices past the head's end read as zeros and are not stored);
// 16-bit or fp32 inputs.

#include <stdlib.h>
#include <string.h>

#include "device_common.hpp"
#include "attention_backward.hpp"

namespace areno {
namespace {


constexpr int kBwdWaves = 4;
constexpr int kLanesPerKey = 4;
constexpr int kKeysPerPass = kWave / kLanesPerKey;  // 16
constexpr float kNegInfB = -__builtin_huge_valf();

__device__ __forceinline__ int find_seq(const int32_t* cu, int num_seqs, int64_t token) {
  int lo = 0, hi = num_seqs;
  while (lo + 1 < hi) {
    const int mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(cu[mid]) <= token) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

// The first `valid` (a multiple of 8) of EPL consecutive elements starting at element index idx (a multiple of 8) as
// floats, zeros behind them
template <int EPL>
__device__ __forceinline__ void load_slice(const void* base, int64_t idx, int dtype, int valid, float (&x)[EPL]) {
  if (dtype == ARENO_DT_F32) {
    const float4_t* src = reinterpret_cast<const float4_t*>(static_cast<const float*>(base) + idx);
#pragma unroll
    for (int c = 0; c < EPL / 4; ++c) {
      const float4_t w = 4 * c < valid ? src[c] : float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 4; ++j) x[4 * c + j] = w[j];
    }
  } else {
    const uint4_t* src = reinterpret_cast<const uint4_t*>(static_cast<const uint16_t*>(base) + idx);
#pragma unroll
    for (int c = 0; c < EPL / 8; ++c) {
      const uint4_t w = 8 * c < valid ? src[c] : uint4_t{0u, 0u, 0u, 0u};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (dtype == ARENO_DT_BF16) {
          x[8 * c + 2 * j] = bf16_bits_to_float(w[j] & 0xffffu);
          x[8 * c + 2 * j + 1] = bf16_bits_to_float(w[j] >> 16);
        } else {
          x[8 * c + 2 * j] = f16_bits_to_float(w[j] & 0xffffu);
          x[8 * c + 2 * j + 1] = f16_bits_to_float(w[j] >> 16);
        }
      }
    }
  }
}

// sum over the 4 lanes that share a key / a pair
__device__ __forceinline__ float quad_sum(float x) {
  x += __shfl_xor(x, 1, kWave);
  x += __shfl_xor(x, 2, kWave);
  return x;
}

// sum over the 16 lane groups (lanes with the same position inside their group)
__device__ __forceinline__ float groups_sum(float x) {
#pragma unroll
  for (int off = kLanesPerKey; off < kWave; off <<= 1) x += __shfl_xor(x, off, kWave);
  return x;
}

template <int EPL>
__global__ __launch_bounds__(kBwdWaves* kWave) void attention_backward_rows_kernel(BwdParams p) {
  const int D = p.head_dim;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kBwdWaves + (threadIdx.x >> 6);
  if (row >= p.q_tokens * p.q_heads) return;
  const int64_t token = row / p.q_heads;
  const int h = static_cast<int>(row - token * p.q_heads);
  const int kvh = h / (p.q_heads / p.kv_heads);
  const int grp = lane / kLanesPerKey;
  const int sub = lane % kLanesPerKey;
  const int valid_e = min(max(D - sub * EPL, 0), EPL);  // elements of this lane's slice that lie inside the head
  const int64_t q_base = row * D + sub * EPL;

  if (token >= p.cu_q[p.num_seqs]) {  // rows past the last sequence take part in nothing
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      if (grp == 0 && e < valid_e) store_grad(p.grad_q, q_base + e, 0.0f, p.grad_dtype);
    }
    return;
  }
  const int seq = find_seq(p.cu_q, p.num_seqs, token);
  const int q_pos = (p.ctx != nullptr ? p.ctx[seq] : 0) + static_cast<int>(token - p.cu_q[seq]);
  const int64_t k_begin = p.cu_k[seq];
  const int n_keys = p.cu_k[seq + 1] - p.cu_k[seq];
  const int last = min(q_pos, n_keys - 1);
  const int first = (p.window_left >= 0 && q_pos > p.window_left) ? q_pos - p.window_left : 0;

  float qv[EPL], go[EPL];
  load_slice<EPL>(p.q, q_base, p.dtype, valid_e, qv);
  load_slice<EPL>(p.grad_out, q_base, p.dtype, valid_e, go);
  float d_part = 0.0f;
  {
    float ov[EPL];
    load_slice<EPL>(p.out, q_base, p.dtype, valid_e, ov);
#pragma unroll
    for (int e = 0; e < EPL; ++e) d_part += go[e] * ov[e];
  }
  const float d_row = quad_sum(d_part);  // dO . O

  auto key_base = [&](int pos) { return ((k_begin + pos) * p.kv_heads + kvh) * static_cast<int64_t>(D) + sub * EPL; };

  // ---- pass 1: maximum and sum of the row's exponentials (log2 domain) -------------------------------------------
  float m_g = kNegInfB, l_g = 0.0f;
  for (int base = first; base <= last; base += kKeysPerPass) {
    const int pos = base + grp;
    const bool valid = pos <= last;
    float kx[EPL];
    load_slice<EPL>(p.k, key_base(valid ? pos : last), p.dtype, valid_e, kx);
    float dot = 0.0f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) dot += qv[e] * kx[e];
    const float s = valid ? quad_sum(dot) * p.scale_log2e : kNegInfB;
    const float m_new = fmaxf(m_g, s);
    if (m_new != kNegInfB) {
      l_g = l_g * fast_exp2(m_g - m_new) + fast_exp2(s - m_new);
      m_g = m_new;
    }
  }
  const float m_row = wave_max(m_g);
  const float l_row = wave_sum((sub == 0 && m_g != kNegInfB) ? l_g * fast_exp2(m_g - m_row) : 0.0f);
  const float lse = m_row + __builtin_log2f(l_row);
  if (lane == 0) {
    p.row_stats[row * 2] = lse;
    p.row_stats[row * 2 + 1] = d_row;
  }

  // ---- pass 2: dQ = scale * sum_j P_j (dO . V_j - dO . O) K_j -----------------------------------------------------
  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.0f;
  for (int base = first; base <= last; base += kKeysPerPass) {
    const int pos = base + grp;
    const bool valid = pos <= last;
    const int64_t kb = key_base(valid ? pos : last);
    float kx[EPL], vx[EPL];
    load_slice<EPL>(p.k, kb, p.dtype, valid_e, kx);
    load_slice<EPL>(p.v, kb, p.dtype, valid_e, vx);
    float dot = 0.0f, dpv = 0.0f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      dot += qv[e] * kx[e];
      dpv += go[e] * vx[e];
    }
    const float s = quad_sum(dot) * p.scale_log2e;
    const float prob = valid ? fast_exp2(s - lse) : 0.0f;
    const float ds = prob * (quad_sum(dpv) - d_row);
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] += ds * kx[e];
  }
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const float total = groups_sum(acc[e]);
    if (grp == 0 && e < valid_e) store_grad(p.grad_q, q_base + e, total * p.scale, p.grad_dtype);
  }
}

template <int EPL>
__global__ __launch_bounds__(kBwdWaves* kWave) void attention_backward_keys_kernel(BwdParams p) {
  const int D = p.head_dim;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t krow = static_cast<int64_t>(blockIdx.x) * kBwdWaves + (threadIdx.x >> 6);
  if (krow >= p.k_tokens * p.kv_heads) return;
  const int64_t ktoken = krow / p.kv_heads;
  const int kvh = static_cast<int>(krow - ktoken * p.kv_heads);
  const int group = p.q_heads / p.kv_heads;
  const int grp = lane / kLanesPerKey;
  const int sub = lane % kLanesPerKey;
  const int valid_e = min(max(D - sub * EPL, 0), EPL);
  const int64_t k_base = krow * D + sub * EPL;

  float dk[EPL], dv[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) dk[e] = dv[e] = 0.0f;
  if (ktoken < p.cu_k[p.num_seqs]) {
    const int seq = find_seq(p.cu_k, p.num_seqs, ktoken);
    const int pos = static_cast<int>(ktoken - p.cu_k[seq]);
    const int ctx = p.ctx != nullptr ? p.ctx[seq] : 0;
    const int64_t q_begin = p.cu_q[seq];
    const int n_q = p.cu_q[seq + 1] - p.cu_q[seq];
    // queries (by index inside the sequence) that see this key: position >= pos, and <= pos + window
    const int i_lo = max(0, pos - ctx);
    const int i_hi = p.window_left >= 0 ? min(n_q - 1, pos + p.window_left - ctx) : n_q - 1;
    if (i_lo <= i_hi) {
      float kx[EPL], vx[EPL];
      load_slice<EPL>(p.k, k_base, p.dtype, valid_e, kx);
      load_slice<EPL>(p.v, k_base, p.dtype, valid_e, vx);
      const int64_t pairs = static_cast<int64_t>(i_hi - i_lo + 1) * group;
      for (int64_t t0 = 0; t0 < pairs; t0 += kKeysPerPass) {
        const int64_t t = t0 + grp;
        const bool valid = t < pairs;
        const int64_t tc = valid ? t : pairs - 1;
        const int i = i_lo + static_cast<int>(tc / group);
        const int hh = static_cast<int>(tc % group);
        const int64_t row = (q_begin + i) * p.q_heads + kvh * group + hh;
        float qv[EPL], go[EPL];
        load_slice<EPL>(p.q, row * D + sub * EPL, p.dtype, valid_e, qv);
        load_slice<EPL>(p.grad_out, row * D + sub * EPL, p.dtype, valid_e, go);
        const float lse = p.row_stats[row * 2];
        const float d_row = p.row_stats[row * 2 + 1];
        float dot = 0.0f, dpv = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          dot += qv[e] * kx[e];
          dpv += go[e] * vx[e];
        }
        const float s = quad_sum(dot) * p.scale_log2e;
        const float prob = valid ? fast_exp2(s - lse) : 0.0f;
        const float ds = prob * (quad_sum(dpv) - d_row);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          dv[e] += prob * go[e];
          dk[e] += ds * qv[e];
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const float tk = groups_sum(dk[e]);
    const float tv = groups_sum(dv[e]);
    if (grp == 0 && e < valid_e) {
      store_grad(p.grad_k, k_base + e, tk * p.scale, p.grad_dtype);
      store_grad(p.grad_v, k_base + e, tv, p.grad_dtype);
    }
  }
}

typedef void (*bwd_fn)(BwdParams);

// the narrowest per-lane slice whose four lanes cover the head
bwd_fn rows_kernel_for(int head_dim) {
  if (head_dim <= 0 || head_dim > 256 || head_dim % 8 != 0) return nullptr;
  if (head_dim <= 64) return attention_backward_rows_kernel<16>;
  if (head_dim <= 128) return attention_backward_rows_kernel<32>;
  if (head_dim <= 192) return attention_backward_rows_kernel<48>;
  return attention_backward_rows_kernel<64>;
}

bwd_fn keys_kernel_for(int head_dim) {
  if (head_dim <= 0 || head_dim > 256 || head_dim % 8 != 0) return nullptr;
  if (head_dim <= 64) return attention_backward_keys_kernel<16>;
  if (head_dim <= 128) return attention_backward_keys_kernel<32>;
  if (head_dim <= 192) return attention_backward_keys_kernel<48>;
  return attention_backward_keys_kernel<64>;
}

}  // namespace
}  // namespace areno

extern "C" size_t areno_hip_attention_backward_workspace_bytes(int64_t q_tokens, int32_t q_heads) {
  if (q_tokens <= 0 || q_heads <= 0) return 0;
  return static_cast<size_t>(q_tokens) * q_heads * 2 * sizeof(float);
}

extern "C" int areno_hip_attention_backward(const void* grad_out, const void* q, const void* k, const void* v,
                                            const void* out, float* grad_q, float* grad_k, float* grad_v,
                                            int32_t dtype, int64_t q_tokens, int64_t k_tokens, int32_t q_heads,
                                            int32_t kv_heads, int32_t head_dim, const int32_t* cu_seqlens_q,
                                            const int32_t* cu_seqlens_k, const int32_t* context_lens, int32_t num_seqs,
                                            int32_t window_left, float softmax_scale, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  return areno_hip_attention_backward_typed(grad_out, q, k, v, out, grad_q, grad_k, grad_v, ARENO_DT_F32, dtype, q_tokens,
                                            k_tokens, q_heads, kv_heads, head_dim, cu_seqlens_q, cu_seqlens_k,
                                            context_lens, num_seqs, window_left, softmax_scale, workspace,
                                            workspace_bytes, stream);
}

extern "C" int areno_hip_attention_backward_typed(const void* grad_out, const void* q, const void* k, const void* v,
                                                  const void* out, void* grad_q, void* grad_k, void* grad_v,
                                                  int32_t grad_dtype, int32_t dtype, int64_t q_tokens, int64_t k_tokens,
                                                  int32_t q_heads, int32_t kv_heads, int32_t head_dim,
                                                  const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                                  const int32_t* context_lens, int32_t num_seqs, int32_t window_left,
                                                  float softmax_scale, void* workspace, size_t workspace_bytes,
                                                  void* stream) {
  using namespace areno;
  const char* op = "areno_hip_attention_backward";
  if (grad_dtype != ARENO_DT_F32 && grad_dtype != dtype)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: gradients come in f32 or in the inputs' type", op);
  if (q_tokens < 0 || k_tokens < 0 || num_seqs < 1 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range or q_heads not a multiple of kv_heads", op);
  if (dtype != ARENO_DT_F32 && dtype != ARENO_DT_F16 && dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: dtype must be f32, f16 or bf16", op);
  bwd_fn rows = rows_kernel_for(head_dim);
  bwd_fn keys = keys_kernel_for(head_dim);
  if (rows == nullptr || keys == nullptr)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim %d (multiples of 8 up to 256 are built)", op, head_dim);
  if (q_tokens == 0 && k_tokens == 0) return ARENO_OK;
  if (grad_out == nullptr || q == nullptr || k == nullptr || v == nullptr || out == nullptr || grad_q == nullptr ||
      grad_k == nullptr || grad_v == nullptr || cu_seqlens_q == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: tensor pointer is NULL", op);
  for (const void* ptr : {grad_out, q, k, v, out, static_cast<const void*>(grad_q), static_cast<const void*>(grad_k),
                          static_cast<const void*>(grad_v)}) {
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return fail(ARENO_ERR_UNSUPPORTED, "%s: tensors must be 16-byte aligned", op);
  }
  const size_t need = areno_hip_attention_backward_workspace_bytes(q_tokens, q_heads);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need))
    return fail(ARENO_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", op, need, workspace_bytes);
  const int64_t q_rows = q_tokens * q_heads;
  const int64_t k_rows = k_tokens * kv_heads;
  if ((q_rows + kBwdWaves - 1) / kBwdWaves > 0x7fffffffLL || (k_rows + kBwdWaves - 1) / kBwdWaves > 0x7fffffffLL)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: too many rows", op);

  BwdParams p;
  p.grad_out = grad_out;
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.grad_q = grad_q;
  p.grad_k = grad_k;
  p.grad_v = grad_v;
  p.row_stats = static_cast<float*>(workspace);
  p.cu_q = cu_seqlens_q;
  p.cu_k = cu_seqlens_k != nullptr ? cu_seqlens_k : cu_seqlens_q;
  p.ctx = context_lens;
  p.q_tokens = q_tokens;
  p.k_tokens = k_tokens;
  p.num_seqs = num_seqs;
  p.q_heads = q_heads;
  p.kv_heads = kv_heads;
  p.window_left = window_left;
  p.head_dim = head_dim;
  p.dtype = dtype;
  p.grad_dtype = grad_dtype;
  p.scale = softmax_scale;
  p.scale_log2e = softmax_scale * kLog2e;
  // 16-bit inputs at head dims 64 and 128 run on the matrix cores (ARENO_BACKWARD_KERNEL=valu: a diagnosis switch
  // that keeps them on the kernels below)
  static const bool valu_only = [] {
    const char* e = getenv("ARENO_BACKWARD_KERNEL");
    return e != nullptr && strcmp(e, "valu") == 0;
  }();
  if (!valu_only) {
    const int rc = launch_attention_backward_mfma(p, stream);
    if (rc != ARENO_ERR_UNSUPPORTED) return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (q_rows > 0) {
    hipLaunchKernelGGL(rows, dim3(static_cast<unsigned>((q_rows + kBwdWaves - 1) / kBwdWaves)), dim3(kBwdWaves * kWave), 0,
                       s, p);
    if (int rc = check_launch(op)) return rc;
  }
  if (k_rows > 0) {
    hipLaunchKernelGGL(keys, dim3(static_cast<unsigned>((k_rows + kBwdWaves - 1) / kBwdWaves)), dim3(kBwdWaves * kWave), 0,
                       s, p);
    if (int rc = check_launch(op)) return rc;
  }
  return ARENO_OK;
}
