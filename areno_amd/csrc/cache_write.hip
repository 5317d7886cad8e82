// Quantize-and-scatter KV-cache write for gfx950.
//
// One wave64 owns one (token, kv head) row of K or V: it loads the row, finds the row's
// abs-max with a wave reduction, derives the per-row scale, converts to int8 / OCP e4m3fn
// codes (or copies, for an unquantized cache) and stores codes and scale at the paged
// address.  Two addressing modes share the kernel:
//   explicit  (block_ids[t], block_offsets[t])                  -- prefill store,
//             areno/engine/layers/attention_backend/infer.py:245-263 in the reference
//   decode    (block_table[b, L_b / bs], L_b % bs)              -- single-token append,
//             areno/accel/csrc/attention.cu:526-553
//
// Quantizer closed forms (bit-exact contract; IEEE fp32 division, round half to even):
//   int8: s = fp16(min(absmax / 127, 65504)); s == 0 -> 1; code = clamp(rint(x / float(s)), -127, 127)
//   fp8 : s = absmax / 448 (fp32);            s == 0 -> 1; code = e4m3fn(clamp(x / s, -448, 448))
// The work is launch-latency bound for decode (B * Hkv rows) and a plain streaming copy for
// prefill; no LDS is needed.

#include "cache_row_quant.hpp"

namespace areno {
namespace {

struct WriteParams {
  const void* src[2];  // k, v
  void* cache[2];
  void* scale[2];
  const int64_t* block_ids;
  const int64_t* block_offsets;
  const int32_t* block_table;
  const int32_t* cache_seqlens;
  int64_t tokens;
  int64_t num_blocks;
  int32_t max_blocks;
  int32_t block_size;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t in_dtype;
  int32_t cache_dtype;
  int32_t scale_dtype;
};

constexpr int kRowsPerBlock = 4;  // one wave per row

__global__ __launch_bounds__(kRowsPerBlock* kWave) void cache_write_kernel(WriteParams p) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= p.tokens * p.kv_heads) return;
  const int which = blockIdx.y;  // 0 = K, 1 = V
  const int64_t token = row / p.kv_heads;
  const int head = static_cast<int>(row - token * p.kv_heads);

  int64_t blk, slot;
  if (p.block_ids != nullptr) {
    blk = p.block_ids[token];
    slot = p.block_offsets[token];
  } else {
    const int64_t pos = p.cache_seqlens[token];
    const int64_t col = pos / p.block_size;
    if (pos < 0 || col >= p.max_blocks) return;
    slot = pos - col * p.block_size;
    blk = p.block_table[token * p.max_blocks + col];
  }
  if (blk < 0 || blk >= p.num_blocks || slot < 0 || slot >= p.block_size) return;

  const int d = p.head_dim;
  const int64_t src_base = row * d;
  const int64_t dst_row = (blk * p.block_size + slot) * p.kv_heads + head;
  const int64_t dst_base = dst_row * d;
  const void* src = p.src[which];
  void* dst = p.cache[which];

  float x[kMaxPerLane];
#pragma unroll
  for (int e = 0; e < kMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    x[e] = idx < d ? load_as_float(src, src_base + idx, p.in_dtype) : 0.0f;
  }

  if (is_quantized_dtype(p.cache_dtype)) {
    quantize_store_row(x, lane, d, dst_row, dst, p.scale[which], p.cache_dtype, p.scale_dtype);
  } else {
    // same-dtype copy: move raw bits so the stored row is bit-identical to the input row
    if (p.cache_dtype == ARENO_DT_F32) {
      const uint32_t* s32 = static_cast<const uint32_t*>(src);
      uint32_t* d32 = static_cast<uint32_t*>(dst);
      for (int idx = lane; idx < d; idx += kWave) d32[dst_base + idx] = s32[src_base + idx];
    } else {
      const uint16_t* s16 = static_cast<const uint16_t*>(src);
      uint16_t* d16 = static_cast<uint16_t*>(dst);
      for (int idx = lane; idx < d; idx += kWave) d16[dst_base + idx] = s16[src_base + idx];
    }
  }
}

// The common shapes (16-bit rows, head_dim = 8 LPR with LPR a power of two up to 64): a row is held by LPR adjacent
// lanes with 8 consecutive elements each, so a wave moves 64 / LPR rows with 16-byte loads and 8- or 16-byte stores
// instead of one row with one element per lane.  Same closed forms, same bits (store_row_slice).
template <int LPR>
__global__ __launch_bounds__(kRowsPerBlock* kWave) void cache_write_rows_kernel(WriteParams p) {
  constexpr int D = LPR * 8;
  constexpr int kRowsPerWave = kWave / LPR;
  const int lane = threadIdx.x & (kWave - 1);
  const int sub = lane % LPR;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (threadIdx.x >> 6);
  const int64_t total = p.tokens * p.kv_heads;
  const int64_t row_raw = wave_id * kRowsPerWave + lane / LPR;
  const bool live = row_raw < total;
  const int64_t row = live ? row_raw : total - 1;  // idle lane groups shadow the last row and store nothing
  const int which = blockIdx.y;                    // 0 = K, 1 = V
  const int64_t token = row / p.kv_heads;
  const int head = static_cast<int>(row - token * p.kv_heads);

  const uint4_t raw = *reinterpret_cast<const uint4_t*>(static_cast<const char*>(p.src[which]) + (row * D + sub * 8) * 2);
  int64_t blk, slot;
  bool ok = live;
  if (p.block_ids != nullptr) {
    blk = p.block_ids[token];
    slot = p.block_offsets[token];
  } else {
    const int64_t pos = p.cache_seqlens[token];
    const int64_t col = pos / p.block_size;
    ok = ok && pos >= 0 && col < p.max_blocks;
    slot = pos - col * p.block_size;
    blk = ok ? p.block_table[token * p.max_blocks + col] : 0;
  }
  ok = ok && blk >= 0 && blk < p.num_blocks && slot >= 0 && slot < p.block_size;

  float x[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t word = raw[j];
    if (p.in_dtype == ARENO_DT_BF16) {
      x[2 * j] = bf16_bits_to_float(word & 0xffffu);
      x[2 * j + 1] = bf16_bits_to_float(word >> 16);
    } else {
      x[2 * j] = f16_bits_to_float(word & 0xffffu);
      x[2 * j + 1] = f16_bits_to_float(word >> 16);
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(x[j]));
  amax = lane_group_max<LPR>(amax);  // every lane of the wave takes part
  if (!ok) return;
  const int64_t dst_row = (blk * p.block_size + slot) * p.kv_heads + head;
  if (is_quantized_dtype(p.cache_dtype)) {
    store_row_slice(x, amax, sub, dst_row, D, p.cache[which], p.scale[which], p.cache_dtype, p.scale_dtype);
  } else {
    // same-dtype copy: the raw bits, so the stored row is bit-identical to the input row
    *reinterpret_cast<uint4_t*>(static_cast<char*>(p.cache[which]) + (dst_row * D + sub * 8) * 2) = raw;
  }
}

typedef void (*write_rows_fn)(WriteParams);
write_rows_fn write_rows_kernel_for(int head_dim, int in_dtype) {
  if (in_dtype != ARENO_DT_F16 && in_dtype != ARENO_DT_BF16) return nullptr;
  switch (head_dim) {
    case 64: return cache_write_rows_kernel<8>;
    case 128: return cache_write_rows_kernel<16>;
    case 256: return cache_write_rows_kernel<32>;
    case 512: return cache_write_rows_kernel<64>;
    default: return nullptr;
  }
}

int validate_cache(const areno_paged_cache* c, const char* op) {
  if (c == nullptr) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: cache descriptor is NULL", op);
  if (c->k == nullptr || c->v == nullptr) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: cache pool pointer is NULL", op);
  if (c->num_blocks <= 0 || c->block_size <= 0 || c->kv_heads <= 0 || c->head_dim <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: cache shape must be positive", op);
  if (c->cache_dtype < ARENO_DT_F32 || c->cache_dtype > ARENO_DT_FP8_E4M3)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: unknown cache dtype %d", op, c->cache_dtype);
  if (is_quantized(c->cache_dtype)) {
    if (c->k_scale == nullptr || c->v_scale == nullptr)
      return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: quantized cache needs k_scale and v_scale", op);
    if (c->scale_dtype != ARENO_DT_F16 && c->scale_dtype != ARENO_DT_F32)
      return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: scale dtype must be f16 or f32", op);
  }
  return ARENO_OK;
}

int launch_write(const areno_paged_cache* cache, const void* k, const void* v, int32_t in_dtype, int64_t tokens,
                 const int64_t* ids, const int64_t* offs, const int32_t* table, int32_t max_blocks,
                 const int32_t* seqlens, void* stream, const char* op) {
  if (int rc = validate_cache(cache, op)) return rc;
  if (tokens < 0) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: negative token count", op);
  if (tokens > 0 && (k == nullptr || v == nullptr))
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: k/v pointer is NULL", op);
  if (cache->head_dim > kMaxPerLane * kWave)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim %d > %d", op, cache->head_dim, kMaxPerLane * kWave);
  if (in_dtype != ARENO_DT_F32 && in_dtype != ARENO_DT_F16 && in_dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: k/v must be f32, f16 or bf16", op);
  if (!is_quantized(cache->cache_dtype) && in_dtype != cache->cache_dtype)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: k/v dtype must equal an unquantized cache's dtype", op);
  if (tokens == 0) return ARENO_OK;
  const int64_t rows = tokens * cache->kv_heads;
  const int64_t blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks > 0x7fffffffLL) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: too many rows", op);

  WriteParams p;
  p.src[0] = k;
  p.src[1] = v;
  p.cache[0] = cache->k;
  p.cache[1] = cache->v;
  p.scale[0] = cache->k_scale;
  p.scale[1] = cache->v_scale;
  p.block_ids = ids;
  p.block_offsets = offs;
  p.block_table = table;
  p.cache_seqlens = seqlens;
  p.tokens = tokens;
  p.num_blocks = cache->num_blocks;
  p.max_blocks = max_blocks;
  p.block_size = cache->block_size;
  p.kv_heads = cache->kv_heads;
  p.head_dim = cache->head_dim;
  p.in_dtype = in_dtype;
  p.cache_dtype = cache->cache_dtype;
  p.scale_dtype = cache->scale_dtype;
  // 16-byte row slices need 16-byte aligned tensors (rows are multiples of 128 bytes there)
  const bool aligned = (reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                        reinterpret_cast<uintptr_t>(cache->k) | reinterpret_cast<uintptr_t>(cache->v)) % 16 == 0;
  const write_rows_fn rows_kernel = aligned ? write_rows_kernel_for(cache->head_dim, in_dtype) : nullptr;
  if (rows_kernel != nullptr) {
    const int rows_per_wave = kWave / (cache->head_dim / 8);
    const int64_t waves = (rows + rows_per_wave - 1) / rows_per_wave;
    const int64_t wgs = (waves + kRowsPerBlock - 1) / kRowsPerBlock;
    hipLaunchKernelGGL(rows_kernel, dim3(static_cast<unsigned>(wgs), 2), dim3(kRowsPerBlock * kWave), 0,
                       static_cast<hipStream_t>(stream), p);
    return check_launch(op);
  }
  hipLaunchKernelGGL(cache_write_kernel, dim3(static_cast<unsigned>(blocks), 2), dim3(kRowsPerBlock * kWave), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}

}  // namespace

int validate_paged_cache(const areno_paged_cache* c, const char* op) { return validate_cache(c, op); }

}  // namespace areno

extern "C" int areno_hip_cache_write(const areno_paged_cache* cache, const void* k, const void* v, int32_t in_dtype,
                                     int64_t tokens, const int64_t* block_ids, const int64_t* block_offsets,
                                     void* stream) {
  if (tokens > 0 && (block_ids == nullptr || block_offsets == nullptr))
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "areno_hip_cache_write: block_ids/block_offsets is NULL");
  return areno::launch_write(cache, k, v, in_dtype, tokens, block_ids, block_offsets, nullptr, 0, nullptr, stream,
                             "areno_hip_cache_write");
}

extern "C" int areno_hip_cache_write_decode(const areno_paged_cache* cache, const void* k_update, const void* v_update,
                                            int32_t in_dtype, int32_t batch, const int32_t* block_table,
                                            int32_t max_blocks, const int32_t* cache_seqlens, void* stream) {
  if (batch > 0 && (block_table == nullptr || cache_seqlens == nullptr || max_blocks <= 0))
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "areno_hip_cache_write_decode: block_table/cache_seqlens missing");
  return areno::launch_write(cache, k_update, v_update, in_dtype, batch, nullptr, nullptr, block_table, max_blocks,
                             cache_seqlens, stream, "areno_hip_cache_write_decode");
}
