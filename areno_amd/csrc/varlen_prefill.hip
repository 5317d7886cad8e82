// Causal varlen attention over new tokens, either against packed K/V (the reference's
// varlen_causal_attention_forward_kernel, areno/accel/csrc/attention.cu:145-242) or against
// paged, optionally quantized KV with a cached context (this build's paged prefill).
//
// Generic kernel: one wave64 per (query token, q head); lanes split the head dimension, keys are
// visited one at a time with the reference's online-softmax recurrence in fp32.  It accepts every
// dtype / head_dim <= 512 / head ratio and is the fallback for shapes the MFMA kernel does not cover.

#include "device_common.hpp"

namespace areno {

int validate_paged_cache(const areno_paged_cache* c, const char* op);

namespace {

constexpr int kMaxPerLane = 8;
constexpr float kNegInfF = -__builtin_huge_valf();

struct VarlenParams {
  const void* q;
  const void* k;  // packed K (tokens, kv_heads, d) or paged pool
  const void* v;
  const void* k_scale;
  const void* v_scale;
  void* out;
  const int32_t* cu_seqlens;    // (num_seqs + 1)
  const int32_t* context_lens;  // (num_seqs) or nullptr (packed mode: context 0)
  const int32_t* block_table;   // nullptr in packed mode
  int64_t tokens;
  int32_t num_seqs;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t block_size;
  int32_t max_blocks;
  int32_t window_left;
  int32_t q_dtype;
  int32_t kv_dtype;
  int32_t scale_dtype;
  float scale_log2e;
};

// last sequence s with cu_seqlens[s] <= token (binary search, as attention.cu:26-38)
__device__ __forceinline__ int find_sequence(const int32_t* cu, int num_seqs, int64_t token) {
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

constexpr int kRowsPerBlock = 4;

__global__ __launch_bounds__(kRowsPerBlock* kWave) void varlen_generic_kernel(VarlenParams p) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= p.tokens * p.q_heads) return;
  const int64_t token = row / p.q_heads;
  const int h = static_cast<int>(row - token * p.q_heads);
  const int kvh = h / (p.q_heads / p.kv_heads);
  const int d = p.head_dim;
  const int64_t out_base = row * d;

  const int seq = find_sequence(p.cu_seqlens, p.num_seqs, token);
  const int64_t seq_start = p.cu_seqlens[seq];
  if (token >= p.cu_seqlens[p.num_seqs]) {  // rows past the last sequence: defined output, no keys
    for (int idx = lane; idx < d; idx += kWave) store_from_float(p.out, out_base + idx, p.q_dtype, 0.0f);
    return;
  }
  const int local_q = static_cast<int>(token - seq_start);
  const int ctx = p.context_lens != nullptr ? p.context_lens[seq] : 0;
  const int q_pos = ctx + local_q;  // absolute position of the query inside its sequence
  const int first_key = (p.window_left >= 0 && q_pos > p.window_left) ? q_pos - p.window_left : 0;
  const bool quant = p.kv_dtype == ARENO_DT_I8 || p.kv_dtype == ARENO_DT_FP8_E4M3;

  float q[kMaxPerLane], acc[kMaxPerLane];
#pragma unroll
  for (int e = 0; e < kMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    q[e] = idx < d ? load_as_float(p.q, out_base + idx, p.q_dtype) : 0.0f;
    acc[e] = 0.0f;
  }
  float m = kNegInfF, l = 0.0f;
  for (int key = first_key; key <= q_pos; ++key) {
    int64_t r;
    if (p.block_table != nullptr) {
      const int col = key / p.block_size;
      const int slot = key - col * p.block_size;
      const int64_t blk = p.block_table[static_cast<int64_t>(seq) * p.max_blocks + col];
      r = (blk * p.block_size + slot) * p.kv_heads + kvh;
    } else {
      r = (seq_start + key) * p.kv_heads + kvh;
    }
    float dot = 0.0f;
    float v[kMaxPerLane];
#pragma unroll
    for (int e = 0; e < kMaxPerLane; ++e) {
      const int idx = lane + e * kWave;
      if (idx < d) {
        dot += q[e] * load_as_float(p.k, r * d + idx, p.kv_dtype);
        v[e] = load_as_float(p.v, r * d + idx, p.kv_dtype);
      } else {
        v[e] = 0.0f;
      }
    }
    dot = wave_sum(dot);
    float ks = 1.0f, vs = 1.0f;
    if (quant) {
      ks = load_scale(p.k_scale, r, p.scale_dtype);
      vs = load_scale(p.v_scale, r, p.scale_dtype);
    }
    const float s = dot * ks * p.scale_log2e;
    const float m_new = fmaxf(m, s);
    const float alpha = fast_exp2(m - m_new);
    const float beta = fast_exp2(s - m_new);
    l = l * alpha + beta;
    m = m_new;
    const float bv = beta * vs;
#pragma unroll
    for (int e = 0; e < kMaxPerLane; ++e) acc[e] = acc[e] * alpha + bv * v[e];
  }
#pragma unroll
  for (int e = 0; e < kMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    if (idx < d) store_from_float(p.out, out_base + idx, p.q_dtype, acc[e] / l);
  }
}

int launch_generic(const VarlenParams& p, void* stream, const char* op) {
  const int64_t rows = p.tokens * p.q_heads;
  const int64_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks > 0x7fffffffLL) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: too many rows", op);
  hipLaunchKernelGGL(varlen_generic_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kRowsPerBlock * kWave), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}

}  // namespace

// Defined in prefill_mfma.hip: returns ARENO_ERR_UNSUPPORTED when the shape has no MFMA kernel.
int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* workspace, size_t workspace_bytes, void* stream);
size_t prefill_mfma_workspace_bytes(int32_t kv_heads, int32_t head_dim);

}  // namespace areno

extern "C" size_t areno_hip_prefill_workspace_bytes(int32_t kv_heads, int32_t head_dim) {
  return areno::prefill_mfma_workspace_bytes(kv_heads, head_dim);
}

extern "C" int areno_hip_varlen_attention(const void* q, const void* k, const void* v, void* out, int32_t dtype,
                                          int64_t tokens, int32_t q_heads, int32_t kv_heads, int32_t head_dim,
                                          const int32_t* cu_seqlens, int32_t num_seqs, int32_t window_left,
                                          float softmax_scale, void* workspace, size_t workspace_bytes,
                                          void* stream) {
  using namespace areno;
  const char* op = "areno_hip_varlen_attention";
  if (q == nullptr || k == nullptr || v == nullptr || out == nullptr || cu_seqlens == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", op);
  if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || num_seqs < 1)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
  if (q_heads % kv_heads != 0) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: q heads must be divisible by kv heads", op);
  if (dtype != ARENO_DT_F32 && dtype != ARENO_DT_F16 && dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: dtype must be f32, f16 or bf16", op);
  if (head_dim > kMaxPerLane * kWave) return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim %d > 512", op, head_dim);
  if (tokens == 0) return ARENO_OK;
  {
    // packed K/V described as a one-block "cache" for the MFMA kernel (it addresses rows directly in this mode)
    areno_paged_cache packed = {};
    packed.k = const_cast<void*>(k);
    packed.v = const_cast<void*>(v);
    packed.num_blocks = 1;
    packed.block_size = 1;
    packed.kv_heads = kv_heads;
    packed.head_dim = head_dim;
    packed.cache_dtype = dtype;
    packed.scale_dtype = ARENO_DT_F32;
    const int rc = launch_prefill_mfma(&packed, q, out, dtype, tokens, q_heads, num_seqs, nullptr, 1, cu_seqlens,
                                       nullptr, window_left, softmax_scale, workspace, workspace_bytes, stream);
    if (rc != ARENO_ERR_UNSUPPORTED) return rc;
  }
  VarlenParams p = {};
  p.q = q;
  p.k = k;
  p.v = v;
  p.out = out;
  p.cu_seqlens = cu_seqlens;
  p.tokens = tokens;
  p.num_seqs = num_seqs;
  p.q_heads = q_heads;
  p.kv_heads = kv_heads;
  p.head_dim = head_dim;
  p.block_size = 1;
  p.window_left = window_left;
  p.q_dtype = dtype;
  p.kv_dtype = dtype;
  p.scale_log2e = softmax_scale * kLog2e;
  return launch_generic(p, stream, op);
}

extern "C" int areno_hip_paged_varlen_prefill(const areno_paged_cache* cache, const void* q, void* out,
                                              int32_t q_dtype, int64_t tokens, int32_t q_heads, int32_t num_seqs,
                                              const int32_t* block_table, int32_t max_blocks,
                                              const int32_t* cu_seqlens_q, const int32_t* context_lens,
                                              int32_t window_left, float softmax_scale, void* workspace,
                                              size_t workspace_bytes, void* stream) {
  using namespace areno;
  const char* op = "areno_hip_paged_varlen_prefill";
  if (int rc = validate_paged_cache(cache, op)) return rc;
  if (q == nullptr || out == nullptr || block_table == nullptr || cu_seqlens_q == nullptr || context_lens == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", op);
  if (tokens < 0 || q_heads <= 0 || num_seqs < 1 || max_blocks <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
  if (q_heads % cache->kv_heads != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: q heads must be divisible by kv heads", op);
  if (q_dtype != ARENO_DT_F32 && q_dtype != ARENO_DT_F16 && q_dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: q must be f32, f16 or bf16", op);
  if (!is_quantized(cache->cache_dtype) && cache->cache_dtype != q_dtype)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: q dtype must equal an unquantized cache's dtype", op);
  if (cache->head_dim > kMaxPerLane * kWave)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim %d > 512", op, cache->head_dim);
  if (tokens == 0) return ARENO_OK;

  const int rc = launch_prefill_mfma(cache, q, out, q_dtype, tokens, q_heads, num_seqs, block_table, max_blocks,
                                     cu_seqlens_q, context_lens, window_left, softmax_scale, workspace, workspace_bytes,
                                     stream);
  if (rc != ARENO_ERR_UNSUPPORTED) return rc;

  VarlenParams p = {};
  p.q = q;
  p.k = cache->k;
  p.v = cache->v;
  p.k_scale = cache->k_scale;
  p.v_scale = cache->v_scale;
  p.out = out;
  p.cu_seqlens = cu_seqlens_q;
  p.context_lens = context_lens;
  p.block_table = block_table;
  p.tokens = tokens;
  p.num_seqs = num_seqs;
  p.q_heads = q_heads;
  p.kv_heads = cache->kv_heads;
  p.head_dim = cache->head_dim;
  p.block_size = cache->block_size;
  p.max_blocks = max_blocks;
  p.window_left = window_left;
  p.q_dtype = q_dtype;
  p.kv_dtype = cache->cache_dtype;
  p.scale_dtype = cache->scale_dtype;
  p.scale_log2e = softmax_scale * kLog2e;
  return launch_generic(p, stream, op);
}
