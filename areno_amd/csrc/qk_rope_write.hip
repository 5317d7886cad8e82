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
// global access is 16 bytes wide; the rotary partner i +- D/2 is the same slot of the lane D/16 away.  The grid is
// three runs of workgroups, one per kind of row, so a wave's rows are all of one kind and each kind runs code of its
// own: a q row computes no abs-max and no codes, a v row no norm and no rotation, and which tensor a row comes from
// is a scalar.  The cache rows use the closed forms of areno_hip_cache_write's quantizer, so the pages hold exactly
// quantize(k_out) and quantize(v).  Bound: HBM streaming, T * (Hq + 2 Hkv) * D elements in, T * (Hq + Hkv) * D out
// plus the pages; the vector ALU is what the kernel actually waits for (the roundings of every product to the
// activation dtype, which the eager ops of the reference imply, are most of its instructions).

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
  // Per-token rotary rows from areno_hip_rope_rows ([tokens][2][D] float: the cosines rounded to the activation dtype,
  // then the sines, rounded and with rotate_half's sign on them), or null: the kernel then takes a token's position,
  // fetches its rows of the tables and rounds them itself, once per (token, head) row.
  const float* rope_rows;
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
  uint32_t q_blocks;   // workgroups of q rows; they come first in the grid
  uint32_t kv_blocks;  // workgroups of k rows, then as many of v rows
};

// x rounded to the activation dtype, as float
__device__ __forceinline__ float round_to(float x, int dtype) {
  return dtype == ARENO_DT_BF16 ? bf16_bits_to_float(float_to_bf16_bits(x)) : f16_bits_to_float(float_to_f16_bits(x));
}

// Two values rounded to the activation dtype: the packed pair is returned and the floats are replaced by the rounded
// values (one packed conversion and two unpacking steps for bf16; a caller that only stores the pair pays for the
// conversion alone)
template <int ACT>
__device__ __forceinline__ uint32_t round_pair(float& a, float& b) {
  if constexpr (ACT == ARENO_DT_BF16) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{a, b}, bf16x2_t));
    a = __builtin_bit_cast(float, w << 16);
    b = __builtin_bit_cast(float, w & 0xffff0000u);
    return w;
  } else {
    const uint32_t lo = float_to_f16_bits(a), hi = float_to_f16_bits(b);
    a = f16_bits_to_float(lo);
    b = f16_bits_to_float(hi);
    return lo | (hi << 16);
  }
}

// Row layout: a row of D elements is held by LPR = D / 8 adjacent lanes, 8 consecutive elements (16 bytes of 16-bit
// activations) per lane, so a wave64 carries 64 / LPR rows and every global access is a 16-byte one.  The rotary
// partner of element i (i +- D/2) is the same element slot of lane ^ (LPR / 2).
//
// Exchanges inside a 16-lane row go through the vector ALU's lane-permute modifiers instead of the LDS crossbar:
// lane ^ 1 and lane ^ 2 are quad permutes; after those the four lanes of a quad agree, so mirroring the row's halves
// (lane -> 7 - lane in each 8) and then the row (lane -> 15 - lane) fetch what lane ^ 4 and lane ^ 8 hold; a rotation
// by 8 is lane ^ 8 exactly.
template <int CTRL>
__device__ __forceinline__ float row_permute(float x) {
  // every lane has a source lane in these permutes, so the value for lanes without one is never used; saying so
  // (bound_ctrl) lets the compiler fold the permute into the instruction that consumes it
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
constexpr int kDppQuadXor1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // row_half_mirror
constexpr int kDppMirror = 0x140;      // row_mirror
constexpr int kDppRotate8 = 0x128;     // row_ror:8

// all-reduce over the LPR lanes of a row with `op`, every lane ends with the result (the combination order is that of
// an xor butterfly over masks 1, 2, 4, ...)
template <int LPR, typename Op>
__device__ __forceinline__ float group_reduce(float x, Op op) {
  if constexpr (LPR >= 2) x = op(x, row_permute<kDppQuadXor1>(x));
  if constexpr (LPR >= 4) x = op(x, row_permute<kDppQuadXor2>(x));
  if constexpr (LPR >= 8) x = op(x, row_permute<kDppHalfMirror>(x));
  if constexpr (LPR >= 16) x = op(x, row_permute<kDppMirror>(x));
#pragma unroll
  for (int m = 16; m < LPR; m <<= 1) x = op(x, wave_xor(x, m));
  return x;
}

template <int LPR>
__device__ __forceinline__ float rotary_partner(float x) {
  if constexpr (LPR == 16) {
    return row_permute<kDppRotate8>(x);
  } else {
    return wave_xor(x, LPR / 2);
  }
}

// The rows of one kind (KIND 0: q heads, 1: k heads, 2: v heads) that workgroup `block` of that kind's run takes.
// ACT: the activation dtype (ARENO_DT_F16 / ARENO_DT_BF16): no rounding step branches on it.  The launcher checks that
// rows, element offsets of q / k / v and page rows fit 32 bits, so the index arithmetic is 32-bit, with one division
// per wave (the rows of a wave are consecutive).
template <int LPR, int ACT, int KIND, bool ROWS>
__device__ __forceinline__ void rope_write_rows(const RopeWriteParams& p, uint32_t block) {
  constexpr int D = LPR * 8;
  constexpr int kRowsPerWave = kWave / LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int sub = lane % LPR;  // which 8 elements of the row
  const uint32_t heads = static_cast<uint32_t>(KIND == 0 ? p.q_heads : p.kv_heads);
  const uint32_t total = static_cast<uint32_t>(p.tokens) * heads;
  const uint32_t wave_row = (block * (blockDim.x / kWave) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) * kRowsPerWave;

  // ---- which row: (token, head) of the wave's first row by one scalar division, the lane group's from there --------
  const bool live = wave_row + lane / LPR < total;
  const uint32_t first = min(wave_row, total - 1);  // idle lane groups shadow the last row and store nothing
  const uint32_t ahead = min(static_cast<uint32_t>(lane / LPR), total - 1 - first);
  const uint32_t row = first + ahead;
  uint32_t token = first / heads;
  uint32_t head = first - token * heads + ahead;
  // at most kRowsPerWave - 1 rows further on: one token further when a token has that many heads or more
  const int wraps = heads >= static_cast<uint32_t>(kRowsPerWave) ? 1 : kRowsPerWave - 1;
  for (int i = 0; i < wraps; ++i) {
    const bool wrap = head >= heads;
    head -= wrap ? heads : 0u;
    token += wrap ? 1u : 0u;
  }
  // byte offsets are 32-bit (the launcher's limits), so an access is a scalar base plus a lane's 32-bit offset
  const char* src = static_cast<const char*>(KIND == 0 ? p.q : (KIND == 1 ? p.k : p.v));
  const uint32_t row_bytes = (row * D + sub * 8) * 2u;
  const uint4_t raw = *reinterpret_cast<const uint4_t*>(src + row_bytes);

  void* const cache = KIND == 0 ? nullptr : p.cache[KIND == 2 ? 1 : 0];
  int64_t blk = -1, off = 0;
  if (KIND != 0 && cache != nullptr) {
    blk = *reinterpret_cast<const int64_t*>(reinterpret_cast<const char*>(p.block_ids) + token * 8u);
    off = *reinterpret_cast<const int64_t*>(reinterpret_cast<const char*>(p.block_offsets) + token * 8u);
  }

  float x[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t word = raw[j];
    if (ACT == ARENO_DT_BF16) {
      x[2 * j] = bf16_bits_to_float(word & 0xffffu);
      x[2 * j + 1] = __builtin_bit_cast(float, word & 0xffff0000u);
    } else {
      x[2 * j] = f16_bits_to_float(word & 0xffffu);
      x[2 * j + 1] = f16_bits_to_float(word >> 16);
    }
  }

  if constexpr (KIND != 2) {
    // ---- q and k rows: norm and rotary ----------------------------------------------------------------------------
    const float* cos_row;
    const float* sin_row;
    if constexpr (ROWS) {
      const uint32_t rows_bytes = (token * (2 * D) + sub * 8) * 4u;
      cos_row = reinterpret_cast<const float*>(reinterpret_cast<const char*>(p.rope_rows) + rows_bytes);
      sin_row = cos_row + D;
    } else {
      const int64_t pos = *reinterpret_cast<const int64_t*>(reinterpret_cast<const char*>(p.positions) + token * 8u);
      const uint32_t pc =
          pos < 0 ? 0u : (pos >= p.max_pos ? static_cast<uint32_t>(p.max_pos - 1) : static_cast<uint32_t>(pos));
      const uint32_t table_bytes = (pc * D + sub * 8) * 4u;
      cos_row = reinterpret_cast<const float*>(reinterpret_cast<const char*>(p.cos) + table_bytes);
      sin_row = reinterpret_cast<const float*>(reinterpret_cast<const char*>(p.sin) + table_bytes);
    }
    const float4_t c0 = *reinterpret_cast<const float4_t*>(cos_row);
    const float4_t c1 = *reinterpret_cast<const float4_t*>(cos_row + 4);
    const float4_t s0 = *reinterpret_cast<const float4_t*>(sin_row);
    const float4_t s1 = *reinterpret_cast<const float4_t*>(sin_row + 4);
    const float* weight = KIND == 0 ? p.q_weight : p.k_weight;
    if (weight != nullptr) {
      float sum_sq = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) sum_sq += x[j] * x[j];
      sum_sq = group_reduce<LPR>(sum_sq, [](float a, float b) { return a + b; });
      const float inv = rsqrtf(sum_sq / static_cast<float>(D) + p.eps);
      const float4_t w0 = *reinterpret_cast<const float4_t*>(weight + sub * 8);
      const float4_t w1 = *reinterpret_cast<const float4_t*>(weight + sub * 8 + 4);
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        float a = x[j] * inv * (j < 4 ? w0[j & 3] : w1[j & 3]);
        float b = x[j + 1] * inv * (j < 4 ? w0[(j + 1) & 3] : w1[(j + 1) & 3]);
        round_pair<ACT>(a, b);
        x[j] = a;
        x[j + 1] = b;
      }
    }
    // rotate_half: -x[i + D/2] below D/2, x[i - D/2] above; the sign goes onto the (rounded) sine, which leaves every
    // rounded product what it was
    const uint32_t sign = sub < LPR / 2 ? 0x80000000u : 0u;
    uint32_t packed[4];
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      float ca = j < 4 ? c0[j & 3] : c1[j & 3], cb = j < 4 ? c0[(j + 1) & 3] : c1[(j + 1) & 3];
      float sa = j < 4 ? s0[j & 3] : s1[j & 3], sb = j < 4 ? s0[(j + 1) & 3] : s1[(j + 1) & 3];
      if constexpr (!ROWS) {  // (prepared rows come rounded and signed)
        round_pair<ACT>(ca, cb);  // the tables are cast to the activation dtype first, as the eager ops do
        round_pair<ACT>(sa, sb);
        sa = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, sa) ^ sign);
        sb = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, sb) ^ sign);
      }
      float xa = x[j] * ca, xb = x[j + 1] * cb;
      round_pair<ACT>(xa, xb);
      float ra = rotary_partner<LPR>(x[j]) * sa, rb = rotary_partner<LPR>(x[j + 1]) * sb;
      round_pair<ACT>(ra, rb);
      float ya = xa + ra, yb = xb + rb;
      packed[j / 2] = round_pair<ACT>(ya, yb);
      x[j] = ya;  // read again only by the page store of a k row
      x[j + 1] = yb;
    }
    void* out = KIND == 0 ? p.q_out : p.k_out;
    if (out != nullptr && live)
      *reinterpret_cast<uint4_t*>(static_cast<char*>(out) + row_bytes) = uint4_t{packed[0], packed[1], packed[2], packed[3]};
  }

  if constexpr (KIND != 0) {
    // ---- k and v rows: into the page, through the cache writer's closed forms ------------------------------------
    if (cache == nullptr) return;
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(x[j]));
    amax = group_reduce<LPR>(amax, [](float a, float b) { return fmaxf(a, b); });
    if (!live || blk < 0 || blk >= p.num_blocks || off < 0 || off >= p.block_size) return;
    const uint32_t page_row =
        static_cast<uint32_t>(blk) * static_cast<uint32_t>(p.block_size) + static_cast<uint32_t>(off);
    const int64_t dst_row = static_cast<int64_t>(static_cast<uint64_t>(page_row) * heads + head);
    store_row_slice(x, amax, sub, dst_row, D, cache, p.scale[KIND == 2 ? 1 : 0], p.cache_dtype, p.scale_dtype);
  }
}

template <int LPR, int ACT, bool ROWS>
__global__ __launch_bounds__(256) void qk_rope_write_kernel(RopeWriteParams p) {
  const uint32_t block = blockIdx.x;
  if (block < p.q_blocks) {
    rope_write_rows<LPR, ACT, 0, ROWS>(p, block);
  } else if (block < p.q_blocks + p.kv_blocks) {
    rope_write_rows<LPR, ACT, 1, ROWS>(p, block - p.q_blocks);
  } else {
    rope_write_rows<LPR, ACT, 2, ROWS>(p, block - p.q_blocks - p.kv_blocks);
  }
}

typedef void (*rope_write_fn)(RopeWriteParams);
template <bool ROWS>
rope_write_fn rope_write_lookup(int head_dim, int dtype) {
  const bool bf16 = dtype == ARENO_DT_BF16;
  switch (head_dim) {
    case 64: return bf16 ? qk_rope_write_kernel<8, ARENO_DT_BF16, ROWS> : qk_rope_write_kernel<8, ARENO_DT_F16, ROWS>;
    case 128: return bf16 ? qk_rope_write_kernel<16, ARENO_DT_BF16, ROWS> : qk_rope_write_kernel<16, ARENO_DT_F16, ROWS>;
    case 256: return bf16 ? qk_rope_write_kernel<32, ARENO_DT_BF16, ROWS> : qk_rope_write_kernel<32, ARENO_DT_F16, ROWS>;
    case 512: return bf16 ? qk_rope_write_kernel<64, ARENO_DT_BF16, ROWS> : qk_rope_write_kernel<64, ARENO_DT_F16, ROWS>;
    default: return nullptr;
  }
}

// The rotary rows of a step's tokens, prepared once for all layers: thread (token, 4 elements) fetches the token's
// position, its four cosines and sines, rounds them to the activation dtype (the cast the eager ops make, rotary.py:
// 46-52 in the reference) and puts rotate_half's sign on the sines of the row's first half.
struct RopeRowsParams {
  float* rows;
  const int64_t* positions;
  const float* cos;
  const float* sin;
  int64_t tokens;
  int32_t head_dim;
  int32_t max_pos;
  int32_t dtype;
};
__global__ __launch_bounds__(256) void rope_rows_kernel(RopeRowsParams p) {
  const int64_t quads_per_row = p.head_dim / 4;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= p.tokens * quads_per_row) return;
  const int64_t token = idx / quads_per_row;
  const int e0 = static_cast<int>(idx - token * quads_per_row) * 4;
  const int64_t pos = p.positions[token];
  const int64_t pc = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
  const float4_t c = *reinterpret_cast<const float4_t*>(p.cos + pc * p.head_dim + e0);
  const float4_t s = *reinterpret_cast<const float4_t*>(p.sin + pc * p.head_dim + e0);
  const float sign = e0 < p.head_dim / 2 ? -1.0f : 1.0f;
  float4_t cr, sr;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    cr[j] = round_to(c[j], p.dtype);
    sr[j] = sign * round_to(s[j], p.dtype);
  }
  float* dst = p.rows + token * (2 * p.head_dim) + e0;
  *reinterpret_cast<float4_t*>(dst) = cr;
  *reinterpret_cast<float4_t*>(dst + p.head_dim) = sr;
}

}  // namespace

int64_t g_rope_tokens_per_launch = 0;  // test hook, see areno_hip_debug_set_rope_tokens_per_launch
}  // namespace areno

namespace areno {
namespace {
// rope_rows != nullptr: the prepared rows of the call's tokens stand in for positions / cos / sin / max_pos
int rope_write_impl(const char* op, const areno_paged_cache* cache, const void* q, const void* k, const void* v,
                    void* q_out, void* k_out, int32_t dtype, int64_t tokens, int32_t q_heads, int32_t kv_heads,
                    int32_t head_dim, const int64_t* positions, const float* cos, const float* sin, int32_t max_pos,
                    const float* rope_rows, const float* q_weight, const float* k_weight, float eps,
                    const int64_t* block_ids, const int64_t* block_offsets, void* stream) {
  if (dtype != ARENO_DT_F16 && dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: activations must be f16 or bf16", op);
  if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_pos <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
  if (head_dim != 64 && head_dim != 128 && head_dim != 256 && head_dim != 512)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim must be 64, 128, 256 or 512, got %d", op, head_dim);
  if (tokens == 0) return ARENO_OK;
  if (q == nullptr || k == nullptr || v == nullptr || q_out == nullptr ||
      (rope_rows == nullptr && (positions == nullptr || cos == nullptr || sin == nullptr)))
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", op);
  if (rope_rows != nullptr && reinterpret_cast<uintptr_t>(rope_rows) % 16 != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: rope_rows must be 16-byte aligned", op);
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
  p.rope_rows = rope_rows;
  p.block_ids = block_ids;
  p.block_offsets = block_offsets;
  p.tokens = tokens;
  p.q_heads = q_heads;
  p.kv_heads = kv_heads;
  p.head_dim = head_dim;
  p.max_pos = max_pos;
  p.dtype = dtype;
  p.eps = eps;
  const rope_write_fn fn = rope_rows != nullptr ? rope_write_lookup<true>(head_dim, dtype) : rope_write_lookup<false>(head_dim, dtype);
  if (fn == nullptr) return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim must be 64, 128, 256 or 512, got %d", op, head_dim);
  // The kernel's index arithmetic is 32-bit (rows, element offsets of q / k / v, rotary table offsets, page rows).
  // The table and the pool must fit as they are; a token count past the limits runs as consecutive launches over
  // token ranges.
  const int heads = q_heads + 2 * kv_heads;
  if (heads >= (1 << 16) || static_cast<int64_t>(max_pos) * head_dim >= 0x3fffffffLL)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: %d heads, %d positions x %d are past the kernel's 32-bit indexing", op, heads,
                max_pos, head_dim);
  if (cache != nullptr && cache->num_blocks * cache->block_size > 0xffffffffLL)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: the pool's page rows do not fit 32 bits", op);
  int64_t tokens_per_launch = 0x7fffffffLL / (static_cast<int64_t>(heads) * head_dim) - 1;
  if (tokens_per_launch > (1 << 24) - 1) tokens_per_launch = (1 << 24) - 1;
  // (byte offsets into the prepared rows: 8 * head_dim bytes per token)
  if (rope_rows != nullptr && tokens_per_launch > 0xffffffffLL / (8 * head_dim) - 1) tokens_per_launch = 0xffffffffLL / (8 * head_dim) - 1;
  if (g_rope_tokens_per_launch > 0 && g_rope_tokens_per_launch < tokens_per_launch)
    tokens_per_launch = g_rope_tokens_per_launch;
  if (tokens_per_launch < 1) return fail(ARENO_ERR_UNSUPPORTED, "%s: one token's rows are past 32-bit indexing", op);
  const int rows_per_block = 4 * (kWave / (head_dim / 8));
  const int64_t act_bytes = 2;
  for (int64_t t0 = 0; t0 < tokens; t0 += tokens_per_launch) {
    RopeWriteParams r = p;
    r.tokens = tokens - t0 < tokens_per_launch ? tokens - t0 : tokens_per_launch;
    const int64_t q_off = t0 * q_heads * head_dim * act_bytes, kv_off = t0 * kv_heads * head_dim * act_bytes;
    r.q = static_cast<const char*>(q) + q_off;
    r.k = static_cast<const char*>(k) + kv_off;
    r.v = static_cast<const char*>(v) + kv_off;
    r.q_out = static_cast<char*>(q_out) + q_off;
    r.k_out = k_out == nullptr ? nullptr : static_cast<char*>(k_out) + kv_off;
    r.positions = positions == nullptr ? nullptr : positions + t0;
    r.rope_rows = rope_rows == nullptr ? nullptr : rope_rows + t0 * 2 * head_dim;
    r.block_ids = block_ids == nullptr ? nullptr : block_ids + t0;
    r.block_offsets = block_offsets == nullptr ? nullptr : block_offsets + t0;
    r.q_blocks = static_cast<uint32_t>((r.tokens * q_heads + rows_per_block - 1) / rows_per_block);
    r.kv_blocks = static_cast<uint32_t>((r.tokens * kv_heads + rows_per_block - 1) / rows_per_block);
    hipLaunchKernelGGL(fn, dim3(r.q_blocks + 2 * r.kv_blocks), dim3(256), 0, static_cast<hipStream_t>(stream), r);
    if (int rc = check_launch(op)) return rc;
  }
  return ARENO_OK;
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
  return areno::rope_write_impl("areno_hip_qk_norm_rope_cache_write", cache, q, k, v, q_out, k_out, dtype, tokens, q_heads,
                                kv_heads, head_dim, positions, cos, sin, max_pos, nullptr, q_weight, k_weight, eps,
                                block_ids, block_offsets, stream);
}

extern "C" int areno_hip_qk_norm_rope_cache_write_rows(const areno_paged_cache* cache, const void* q, const void* k,
                                                       const void* v, void* q_out, void* k_out, int32_t dtype,
                                                       int64_t tokens, int32_t q_heads, int32_t kv_heads,
                                                       int32_t head_dim, const float* rope_rows, const float* q_weight,
                                                       const float* k_weight, float eps, const int64_t* block_ids,
                                                       const int64_t* block_offsets, void* stream) {
  const char* op = "areno_hip_qk_norm_rope_cache_write_rows";
  if (rope_rows == nullptr && tokens > 0) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: rope_rows is NULL", op);
  return areno::rope_write_impl(op, cache, q, k, v, q_out, k_out, dtype, tokens, q_heads, kv_heads, head_dim, nullptr,
                                nullptr, nullptr, 1, rope_rows, q_weight, k_weight, eps, block_ids, block_offsets, stream);
}

extern "C" size_t areno_hip_rope_rows_bytes(int64_t tokens, int32_t head_dim) {
  if (tokens < 0 || head_dim <= 0) return 0;
  return static_cast<size_t>(tokens) * 2 * static_cast<size_t>(head_dim) * sizeof(float);
}

extern "C" int areno_hip_rope_rows(float* rows, const int64_t* positions, const float* cos, const float* sin,
                                   int64_t tokens, int32_t head_dim, int32_t max_pos, int32_t dtype, void* stream) {
  using namespace areno;
  const char* op = "areno_hip_rope_rows";
  if (dtype != ARENO_DT_F16 && dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: activations must be f16 or bf16", op);
  if (tokens < 0 || head_dim <= 0 || head_dim % 8 != 0 || max_pos <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: sizes out of range (head_dim must be a multiple of 8)", op);
  if (tokens == 0) return ARENO_OK;
  if (rows == nullptr || positions == nullptr || cos == nullptr || sin == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", op);
  if (reinterpret_cast<uintptr_t>(rows) % 16 != 0 || reinterpret_cast<uintptr_t>(cos) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(sin) % 16 != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: rows / cos / sin must be 16-byte aligned", op);
  RopeRowsParams p = {rows, positions, cos, sin, tokens, head_dim, max_pos, dtype};
  const int64_t threads = tokens * (head_dim / 4);
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(ARENO_ERR_UNSUPPORTED, "%s: too many tokens for one launch", op);
  hipLaunchKernelGGL(rope_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}

// Test hook: caps the tokens one launch of the fused front step takes (0 = only the kernel's own limit), so that the
// walk over token ranges can be exercised at sizes a test can afford.  Returns the previous value.
extern "C" int64_t areno_hip_debug_set_rope_tokens_per_launch(int64_t tokens) {
  const int64_t before = areno::g_rope_tokens_per_launch;
  areno::g_rope_tokens_per_launch = tokens > 0 ? tokens : 0;
  return before;
}
