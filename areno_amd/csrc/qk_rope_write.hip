// The step in front of the attention path, fused: per-head QK RMSNorm, rotary embedding and the quantizing scatter of
// the new K/V rows into the paged cache, in one pass over the projection output.
//
// Reference (one op each, every one a full read and write of its tensor):
//   q = q_norm(q); k = k_norm(k)          areno/engine/layers/attention.py:90-93, kernel
//                                          areno/accel/csrc/normalization.cu:34-56:
//                                          y = dtype(x * rsqrt(mean(x^2) + eps) * w), fp32 arithmetic
//   q, k = rope(q, k, position_ids)       areno/engine/layers/rotary.py:46-52 (rotate_half pairs i with i + D/2):
//                                          dtype(dtype(y * cos) + dtype(rotate_half(y) * sin)) with the fp32 tables
//                                          cast to the activation dtype first -- every product and the sum are
//                                          rounded to the activation dtype, as the eager tensor ops do
//   k_cache[ids, offs] = k; v_cache[...] = v   areno/engine/layers/attention_backend/infer.py:245-263
//
// A (token, head) row is a q head (norm + rope -> q_out), a k head (norm + rope -> k_out and the page) or a v head
// (-> the page).  D / 8 adjacent lanes hold a row, 16 bytes each, so a wave64 carries 64 / (D / 8) rows and every
// global access is 16 bytes wide; the rotary partner i +- D/2 is the same slot of the lane D/16 away.  The cache rows
// use the closed forms of areno_hip_cache_write's quantizer, so the pages hold exactly quantize(k_out) and
// quantize(v).  Bound: HBM streaming, T * (Hq + 2 Hkv) * D elements in, T * (Hq + Hkv) * D out plus the pages.

#include "cache_row_quant.hpp"

namespace areno {

int validate_paged_cache(const areno_paged_cache* c, const char* op);

namespace {

struct RopeWriteParams {
  const void* q;
  const void* k;
  const void* v;
  void* q_out;
  void* k_out;  // may be null
  const float* q_weight;  // [D] or null: no norm on q
  const float* k_weight;  // [D] or null: no norm on k
  const float* cos;       // [max_pos, D]
  const float* sin;
  const int64_t* positions;  // [tokens]
  void* cache[2];            // k, v pools; null pools: no cache write
  void* scale[2];
  const int64_t* block_ids;
  const int64_t* block_offsets;
  int64_t tokens;
  int64_t num_blocks;
  int32_t block_size;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t max_pos;
  int32_t dtype;  // activation dtype: F16 or BF16
  int32_t cache_dtype;
  int32_t scale_dtype;
  float eps;
};

// x rounded to the activation dtype, as float
__device__ __forceinline__ float round_to(float x, int dtype) {
  return dtype == ARENO_DT_BF16 ? bf16_bits_to_float(float_to_bf16_bits(x)) : f16_bits_to_float(float_to_f16_bits(x));
}

// Row layout: a row of D elements is held by LPR = D / 8 adjacent lanes, 8 consecutive elements (16 bytes of 16-bit
// activations) per lane, so a wave64 carries 64 / LPR rows and every global access is a 16-byte one.  The rotary
// partner of element i (i +- D/2) is the same element slot of lane ^ (LPR / 2).
template <int LPR>
__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) x += wave_xor(x, m);
  return x;
}

constexpr int kRowsPerGroup = 1;  // rows a lane group works through (more than one measured slower: 53 vs 36 us at 4)

template <int LPR, int ACT>  // ACT: the activation dtype (ARENO_DT_F16 / ARENO_DT_BF16): no rounding step branches on it
__global__ __launch_bounds__(256) void qk_rope_write_kernel(RopeWriteParams p) {
  constexpr int D = LPR * 8;
  constexpr int kRowsPerWave = kWave / LPR;
  constexpr int R = kRowsPerGroup;
  const int lane = threadIdx.x & (kWave - 1);
  const int sub = lane % LPR;  // which 8 elements of the row
  const int heads = p.q_heads + 2 * p.kv_heads;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + (threadIdx.x >> 6);
  const int64_t total = p.tokens * heads;

  // ---- fetch: row r of this lane group is wave_base + r * rows_per_wave + group, so each load instruction of the
  // wave covers 1 KB of consecutive rows --------------------------------------------------------------------------
  bool live[R];
  int kind[R], head[R];
  int64_t token[R], src_base[R], pos[R];
  uint4_t raw[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row_raw = (wave_id * R + r) * kRowsPerWave + lane / LPR;
    live[r] = row_raw < total;
    const int64_t row = live[r] ? row_raw : total - 1;  // idle lane groups shadow the last row and store nothing
    token[r] = row / heads;
    const int slot = static_cast<int>(row - token[r] * heads);
    kind[r] = slot < p.q_heads ? 0 : (slot < p.q_heads + p.kv_heads ? 1 : 2);  // q, k, v
    head[r] = kind[r] == 0 ? slot : (kind[r] == 1 ? slot - p.q_heads : slot - p.q_heads - p.kv_heads);
    const void* src = kind[r] == 0 ? p.q : (kind[r] == 1 ? p.k : p.v);
    const int src_heads = kind[r] == 0 ? p.q_heads : p.kv_heads;
    src_base[r] = (token[r] * src_heads + head[r]) * D + sub * 8;
    raw[r] = *reinterpret_cast<const uint4_t*>(static_cast<const char*>(src) + src_base[r] * 2);
    pos[r] = p.positions[token[r]];
  }
  float4_t c0[R], c1[R], s0[R], s1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t pc = pos[r] < 0 ? 0 : (pos[r] >= p.max_pos ? p.max_pos - 1 : pos[r]);
    const float* cos_row = p.cos + pc * D + sub * 8;
    const float* sin_row = p.sin + pc * D + sub * 8;
    c0[r] = *reinterpret_cast<const float4_t*>(cos_row);
    c1[r] = *reinterpret_cast<const float4_t*>(cos_row + 4);
    s0[r] = *reinterpret_cast<const float4_t*>(sin_row);
    s1[r] = *reinterpret_cast<const float4_t*>(sin_row + 4);
  }

#pragma unroll
  for (int r = 0; r < R; ++r) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t word = raw[r][j];
      if (ACT == ARENO_DT_BF16) {
        x[2 * j] = bf16_bits_to_float(word & 0xffffu);
        x[2 * j + 1] = bf16_bits_to_float(word >> 16);
      } else {
        x[2 * j] = f16_bits_to_float(word & 0xffffu);
        x[2 * j + 1] = f16_bits_to_float(word >> 16);
      }
    }

    // ---- q and k rows: norm and rotary (selects, not branches, keep every lane in the cross-lane steps) ----------
    const float* weight = kind[r] == 0 ? p.q_weight : (kind[r] == 1 ? p.k_weight : nullptr);
    {
      float sum_sq = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) sum_sq += x[j] * x[j];
      sum_sq = group_sum<LPR>(sum_sq);
      if (weight != nullptr) {
        const float inv = rsqrtf(sum_sq / static_cast<float>(D) + p.eps);
        const float4_t w0 = *reinterpret_cast<const float4_t*>(weight + sub * 8);
        const float4_t w1 = *reinterpret_cast<const float4_t*>(weight + sub * 8 + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          x[j] = round_to(x[j] * inv * w0[j], ACT);
          x[4 + j] = round_to(x[4 + j] * inv * w1[j], ACT);
        }
      }
    }
    float partner[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) partner[j] = wave_xor(x[j], LPR / 2);
    if (kind[r] != 2) {
      const bool low_half = sub < LPR / 2;  // rotate_half: -x[i + D/2] below D/2, x[i - D/2] above
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float c = round_to(j < 4 ? c0[r][j & 3] : c1[r][j & 3], ACT);
        const float sn = round_to(j < 4 ? s0[r][j & 3] : s1[r][j & 3], ACT);
        const float rot = low_half ? -partner[j] : partner[j];
        x[j] = round_to(round_to(x[j] * c, ACT) + round_to(rot * sn, ACT), ACT);
      }
      void* out = kind[r] == 0 ? p.q_out : p.k_out;
      if (out != nullptr && live[r]) {
        const uint4_t packed = {pack_two_16(x[0], x[1], ACT), pack_two_16(x[2], x[3], ACT),
                                pack_two_16(x[4], x[5], ACT), pack_two_16(x[6], x[7], ACT)};
        *reinterpret_cast<uint4_t*>(static_cast<char*>(out) + src_base[r] * 2) = packed;
      }
    }

    // ---- k and v rows: into the page, through the cache writer's closed forms --------------------------------------
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(x[j]));
    amax = lane_group_max<LPR>(amax);
    if (kind[r] == 0 || !live[r]) continue;
    void* cache = p.cache[kind[r] - 1];
    if (cache == nullptr) continue;
    const int64_t blk = p.block_ids[token[r]];
    const int64_t off = p.block_offsets[token[r]];
    if (blk < 0 || blk >= p.num_blocks || off < 0 || off >= p.block_size) continue;
    const int64_t dst_row = (blk * p.block_size + off) * p.kv_heads + head[r];
    store_row_slice(x, amax, sub, dst_row, D, cache, p.scale[kind[r] - 1], p.cache_dtype, p.scale_dtype);
  }
}

typedef void (*rope_write_fn)(RopeWriteParams);
rope_write_fn rope_write_lookup(int head_dim, int dtype) {
  const bool bf16 = dtype == ARENO_DT_BF16;
  switch (head_dim) {
    case 64: return bf16 ? qk_rope_write_kernel<8, ARENO_DT_BF16> : qk_rope_write_kernel<8, ARENO_DT_F16>;
    case 128: return bf16 ? qk_rope_write_kernel<16, ARENO_DT_BF16> : qk_rope_write_kernel<16, ARENO_DT_F16>;
    case 256: return bf16 ? qk_rope_write_kernel<32, ARENO_DT_BF16> : qk_rope_write_kernel<32, ARENO_DT_F16>;
    case 512: return bf16 ? qk_rope_write_kernel<64, ARENO_DT_BF16> : qk_rope_write_kernel<64, ARENO_DT_F16>;
    default: return nullptr;
  }
}

}  // namespace
}  // namespace areno

extern "C" int areno_hip_qk_norm_rope_cache_write(const areno_paged_cache* cache, const void* q, const void* k,
                                                  const void* v, void* q_out, void* k_out, int32_t dtype,
                                                  int64_t tokens, int32_t q_heads, int32_t kv_heads, int32_t head_dim,
                                                  const int64_t* positions, const float* cos, const float* sin,
                                                  int32_t max_pos, const float* q_weight, const float* k_weight,
                                                  float eps, const int64_t* block_ids, const int64_t* block_offsets,
                                                  void* stream) {
  using namespace areno;
  const char* op = "areno_hip_qk_norm_rope_cache_write";
  if (dtype != ARENO_DT_F16 && dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: activations must be f16 or bf16", op);
  if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_pos <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
  if (head_dim != 64 && head_dim != 128 && head_dim != 256 && head_dim != 512)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim must be 64, 128, 256 or 512, got %d", op, head_dim);
  if (tokens == 0) return ARENO_OK;
  if (q == nullptr || k == nullptr || v == nullptr || q_out == nullptr || positions == nullptr || cos == nullptr ||
      sin == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", op);
  RopeWriteParams p = {};
  if (cache != nullptr) {
    if (int rc = validate_paged_cache(cache, op)) return rc;
    if (cache->kv_heads != kv_heads || cache->head_dim != head_dim)
      return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: cache geometry does not match k/v", op);
    if (!is_quantized_dtype(cache->cache_dtype) && cache->cache_dtype != dtype)
      return fail(ARENO_ERR_UNSUPPORTED, "%s: activation dtype must equal an unquantized cache's dtype", op);
    if (block_ids == nullptr || block_offsets == nullptr)
      return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: block_ids/block_offsets is NULL", op);
    p.cache[0] = cache->k;
    p.cache[1] = cache->v;
    p.scale[0] = cache->k_scale;
    p.scale[1] = cache->v_scale;
    p.num_blocks = cache->num_blocks;
    p.block_size = cache->block_size;
    p.cache_dtype = cache->cache_dtype;
    p.scale_dtype = cache->scale_dtype;
  }
  p.q = q;
  p.k = k;
  p.v = v;
  p.q_out = q_out;
  p.k_out = k_out;
  p.q_weight = q_weight;
  p.k_weight = k_weight;
  p.cos = cos;
  p.sin = sin;
  p.positions = positions;
  p.block_ids = block_ids;
  p.block_offsets = block_offsets;
  p.tokens = tokens;
  p.q_heads = q_heads;
  p.kv_heads = kv_heads;
  p.head_dim = head_dim;
  p.max_pos = max_pos;
  p.dtype = dtype;
  p.eps = eps;
  const rope_write_fn fn = rope_write_lookup(head_dim, dtype);
  if (fn == nullptr) return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim must be 64, 128, 256 or 512, got %d", op, head_dim);
  const int64_t rows = tokens * (q_heads + 2 * kv_heads);
  const int rows_per_block = 4 * kRowsPerGroup * (kWave / (head_dim / 8));
  const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
  if (blocks > 0x7fffffffLL) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: too many rows", op);
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}
