/*
 * CPU restatement (plain C, fp32) of the algorithm of the reference's native
 * attention kernels.  TEST INFRASTRUCTURE ONLY: it is the checker for the HIP
 * kernels and the timed CPU baseline, never a product code path.
 *
 * What it follows (areno/accel/csrc/attention.cu in the reference):
 *   oracle_paged_decode_update  <- paged_decode_update_kernel               l.526-553
 *   oracle_paged_decode_split   <- paged_causal_attention_decode_split_kernel  l.555-654
 *   oracle_paged_decode_reduce  <- paged_causal_attention_decode_reduce_kernel l.656-702
 *   oracle_varlen_forward       <- varlen_causal_attention_forward_kernel   l.145-242
 *
 * The recurrence kept from the reference: one key at a time,
 *   new_m = max(m, s); alpha = (l == 0) ? 0 : exp(m - new_m); beta = exp(s - new_m);
 *   l = l*alpha + beta; acc = acc*alpha + beta*v          (l.625-643)
 * a split with no keys leaves (m, l, acc) = (-inf, 0, 0) and the reduce skips
 * partials with l == 0 (l.680-682).  split_size is derived from the full length
 * even under a sliding window (l.588-594).
 *
 * Inputs are fp32 (callers up-cast bf16/fp16 or dequantized caches), so this is
 * the "fp32 reference" the tolerances are stated against.  Parity of this file
 * is pinned in tests/test_oracle_cpu.py against the PyTorch restatement, which
 * in turn is pinned by float64 brute force and SDPA.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  float m;
  float l;
} softmax_state;

static inline void online_step(softmax_state* st, float* acc, const float* v_row, float score, int64_t d_count) {
  const float new_m = fmaxf(st->m, score);
  const float alpha = st->l == 0.0f ? 0.0f : expf(st->m - new_m);
  const float beta = expf(score - new_m);
  st->l = st->l * alpha + beta;
  st->m = new_m;
  for (int64_t d = 0; d < d_count; ++d) acc[d] = acc[d] * alpha + beta * v_row[d];
}

static inline float dot_row(const float* a, const float* b, int64_t n) {
  float s = 0.0f;
  for (int64_t i = 0; i < n; ++i) s += a[i] * b[i];
  return s;
}

void oracle_paged_decode_update(const float* k_update, const float* v_update, float* k_cache, float* v_cache,
                                const int32_t* block_table, const int32_t* cache_seqlens, int64_t batch,
                                int64_t kv_heads, int64_t block_size, int64_t max_blocks, int64_t head_dim) {
  for (int64_t b = 0; b < batch; ++b) {
    const int64_t pos = cache_seqlens[b];
    const int64_t col = pos / block_size;
    const int64_t slot = pos - col * block_size;
    const int64_t blk = block_table[b * max_blocks + col];
    for (int64_t h = 0; h < kv_heads; ++h) {
      const int64_t dst = ((blk * block_size + slot) * kv_heads + h) * head_dim;
      const int64_t src = (b * kv_heads + h) * head_dim;
      memcpy(k_cache + dst, k_update + src, (size_t)head_dim * sizeof(float));
      memcpy(v_cache + dst, v_update + src, (size_t)head_dim * sizeof(float));
    }
  }
}

void oracle_paged_decode_split(const float* q, const float* k_cache, const float* v_cache,
                               const int32_t* block_table, const int32_t* cache_seqlens, float* split_m,
                               float* split_l, float* split_acc, int64_t batch, int64_t q_heads, int64_t kv_heads,
                               int64_t block_size, int64_t max_blocks, int64_t head_dim, int64_t window_left,
                               int64_t num_splits, float softmax_scale) {
  const int64_t group = q_heads / kv_heads;
  const int64_t items = batch * q_heads * num_splits;
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t item = 0; item < items; ++item) {
    const int64_t row = item / num_splits;
    const int64_t split = item - row * num_splits;
    const int64_t b = row / q_heads;
    const int64_t h = row - b * q_heads;
    const int64_t kv_h = h / group;
    const int64_t length = (int64_t)cache_seqlens[b] + 1;
    const int64_t q_pos = length - 1;
    int64_t first_allowed = 0;
    if (window_left >= 0 && q_pos - window_left > 0) first_allowed = q_pos - window_left;
    const int64_t split_size = (length + num_splits - 1) / num_splits;
    int64_t lo = split * split_size;
    int64_t hi = lo + split_size;
    if (hi > length) hi = length;
    if (lo < first_allowed) lo = first_allowed;

    const float* q_row = q + (b * q_heads + h) * head_dim;
    float* acc = split_acc + item * head_dim;
    for (int64_t d = 0; d < head_dim; ++d) acc[d] = 0.0f;
    softmax_state st = {-INFINITY, 0.0f};
    for (int64_t key = lo; key < hi; ++key) {
      const int64_t col = key / block_size;
      const int64_t slot = key - col * block_size;
      const int64_t blk = block_table[b * max_blocks + col];
      const int64_t base = ((blk * block_size + slot) * kv_heads + kv_h) * head_dim;
      const float score = dot_row(q_row, k_cache + base, head_dim) * softmax_scale;
      online_step(&st, acc, v_cache + base, score, head_dim);
    }
    split_m[item] = st.m;
    split_l[item] = st.l;
  }
}

void oracle_paged_decode_reduce(const float* split_m, const float* split_l, const float* split_acc, float* out,
                                int64_t rows, int64_t head_dim, int64_t num_splits) {
#pragma omp parallel for schedule(static)
  for (int64_t row = 0; row < rows; ++row) {
    float* o = out + row * head_dim;
    for (int64_t d = 0; d < head_dim; ++d) o[d] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    for (int64_t s = 0; s < num_splits; ++s) {
      const int64_t item = row * num_splits + s;
      const float part_l = split_l[item];
      if (part_l == 0.0f) continue;
      const float part_m = split_m[item];
      const float new_m = fmaxf(m, part_m);
      const float alpha = l == 0.0f ? 0.0f : expf(m - new_m);
      const float beta = expf(part_m - new_m);
      const float* part = split_acc + item * head_dim;
      for (int64_t d = 0; d < head_dim; ++d) o[d] = o[d] * alpha + part[d] * beta;
      l = l * alpha + part_l * beta;
      m = new_m;
    }
    for (int64_t d = 0; d < head_dim; ++d) o[d] = o[d] / l;
  }
}

/* Whole decode op on fp32 data: update, split, reduce (attention.cu:979-1018). */
int oracle_paged_decode(const float* q, const float* k_update, const float* v_update, float* k_cache, float* v_cache,
                        const int32_t* block_table, const int32_t* cache_seqlens, float* out, int64_t batch,
                        int64_t q_heads, int64_t kv_heads, int64_t block_size, int64_t max_blocks, int64_t head_dim,
                        int64_t window_left, int64_t num_splits, float softmax_scale) {
  const int64_t rows = batch * q_heads;
  float* ws = (float*)malloc((size_t)(rows * num_splits) * (size_t)(head_dim + 2) * sizeof(float));
  if (!ws) return -1;
  float* sm = ws;
  float* sl = sm + rows * num_splits;
  float* sa = sl + rows * num_splits;
  if (k_update && v_update)
    oracle_paged_decode_update(k_update, v_update, k_cache, v_cache, block_table, cache_seqlens, batch, kv_heads,
                               block_size, max_blocks, head_dim);
  oracle_paged_decode_split(q, k_cache, v_cache, block_table, cache_seqlens, sm, sl, sa, batch, q_heads, kv_heads,
                            block_size, max_blocks, head_dim, window_left, num_splits, softmax_scale);
  oracle_paged_decode_reduce(sm, sl, sa, out, rows, head_dim, num_splits);
  free(ws);
  return 0;
}

void oracle_varlen_forward(const float* q, const float* k, const float* v, float* out, const int32_t* cu_seqlens,
                           int64_t total_tokens, int64_t num_seqs, int64_t q_heads, int64_t kv_heads,
                           int64_t head_dim, int64_t window_left, float softmax_scale) {
  const int64_t group = q_heads / kv_heads;
#pragma omp parallel for schedule(dynamic, 8)
  for (int64_t row = 0; row < total_tokens * q_heads; ++row) {
    const int64_t token = row / q_heads;
    const int64_t h = row - token * q_heads;
    const int64_t kv_h = h / group;
    /* last sequence whose start is <= token (the kernel's binary search, l.26-38) */
    int64_t seq = 0;
    for (int64_t s = 0; s < num_seqs; ++s)
      if ((int64_t)cu_seqlens[s] <= token) seq = s;
    const int64_t seq_start = cu_seqlens[seq];
    const int64_t local_q = token - seq_start;
    const int64_t first_key = (window_left >= 0 && local_q > window_left) ? token - window_left : seq_start;
    const float* q_row = q + row * head_dim;
    float* o = out + row * head_dim;
    for (int64_t d = 0; d < head_dim; ++d) o[d] = 0.0f;
    softmax_state st = {-INFINITY, 0.0f};
    for (int64_t key = first_key; key <= token; ++key) {
      const int64_t base = (key * kv_heads + kv_h) * head_dim;
      const float score = dot_row(q_row, k + base, head_dim) * softmax_scale;
      online_step(&st, o, v + base, score, head_dim);
    }
    for (int64_t d = 0; d < head_dim; ++d) o[d] = o[d] / st.l;
  }
}
