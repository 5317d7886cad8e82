// Split-KV GQA paged decode kernels for gfx950 (device code, included by the per-dtype
// instantiation units and by the launcher).
//
// Work decomposition
//   grid  = (chunks, batch, kv-head groups), block = 4 wave64.
//   A workgroup streams one chunk (a fixed number of tokens) of one sequence's pages; wave w owns
//   KV head  z * HW + (w % HW)  and the (w / HW)-th token slice of the chunk, so when kv_heads >= 4 the
//   four waves together read whole pages front to back ([slot][kv_head][D] is contiguous).
//   Every KV byte is read once and applied to all G = q_heads / kv_heads query heads, which are held in
//   registers as packed 16-bit pairs.
// Lane layout inside a wave
//   A K or V row (D elements) is covered by LPT = D * elt_bytes / 16 lanes, each with one 16-byte load;
//   one load instruction therefore fetches TPL = 64 / LPT whole rows (tokens), fully coalesced.
//   QK^T: each lane dots its 16 bytes against the matching slice of the G queries with v_dot2 (two MACs
//   per lane-op, fp32 accumulate) and the LPT partial sums are combined with an xor butterfly.
//   Every group of LPT lanes runs its own online softmax over the tokens it sees (no cross-group traffic in
//   the loop); P.V uses v_dot2 over *token pairs* (two consecutive loads of the same lane), with the
//   per-token V scale folded into P.  The TPL group states are merged once at the end of the wave's slice,
//   then across the waves that share a KV head (through LDS), and one (m, l, acc) partial per
//   (sequence, q head, chunk) goes to the workspace; the reduce kernel merges chunks.
// Dequantisation happens in registers:
//   int8 : byte ^ 0x80 placed in the mantissa of fp16 1024.0 (v_perm with a 0x64 filler) gives 1152 + code
//          exactly; the constant offset is removed algebraically (-1152 * sum(q) on the QK side,
//          -1152 * sum(p) on the PV side), so no per-element subtract is issued.
//   fp8  : v_cvt_pk_f32_fp8 + v_cvt_pkrtz (exact: every e4m3 value is an fp16 value).
//   Per-token scales multiply the score (K) and the probability (V), never the elements.
// Softmax runs in the log2 domain (scores pre-multiplied by log2 e, v_exp_f32).
//
// Semantics follow the reference's split kernel (areno/accel/csrc/attention.cu:555-654): keys
// [first_allowed, L_b], query head h <-> kv head h / G, fp32 accumulation, (m = -inf, l = 0) start state.
#pragma once

#include "device_common.hpp"

namespace areno {

enum KVKind { KV_BF16 = 0, KV_F16 = 1, KV_I8 = 2, KV_FP8 = 3 };

struct DecodeParams {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const void* k_scale;
  const void* v_scale;
  const int32_t* block_table;
  const int32_t* cache_seqlens;
  float* part_ml;   // [batch, q_heads, max_parts, 2]  (m in log2 units, l)
  float* part_acc;  // [batch, q_heads, max_parts, head_dim]
  void* out;
  int32_t batch;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t block_size;
  int32_t bs_shift;  // log2(block_size) or -1
  int32_t max_blocks;
  int32_t window_left;
  int32_t chunk;      // tokens per chunk
  int32_t max_parts;  // chunks per row in the workspace
  int32_t q_dtype;
  int32_t cache_dtype;
  int32_t scale_dtype;
  int32_t group;         // q heads per kv head actually present (<= template G)
  int32_t heads_per_wg;  // HW in {1, 2, 4}
  float scale_log2e;     // softmax_scale * log2(e)
};

constexpr int kDecodeThreads = 256;
constexpr float kNegInf = -__builtin_huge_valf();

template <int KIND>
struct KVTraits;

template <>
struct KVTraits<KV_BF16> {
  static constexpr int kBytes = 2;
  static constexpr bool kQuant = false;
  using pair_t = bf16x2_t;
};
template <>
struct KVTraits<KV_F16> {
  static constexpr int kBytes = 2;
  static constexpr bool kQuant = false;
  using pair_t = half2_t;
};
template <>
struct KVTraits<KV_I8> {
  static constexpr int kBytes = 1;
  static constexpr bool kQuant = true;
  using pair_t = half2_t;
};
template <>
struct KVTraits<KV_FP8> {
  static constexpr int kBytes = 1;
  static constexpr bool kQuant = true;
  using pair_t = half2_t;
};

__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
__device__ __forceinline__ float dot2(bf16x2_t a, bf16x2_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
}

template <typename P>
__device__ __forceinline__ P make_pair(float lo, float hi);
template <>
__device__ __forceinline__ half2_t make_pair<half2_t>(float lo, float hi) {
  half2_t r;
  r.x = static_cast<_Float16>(lo);
  r.y = static_cast<_Float16>(hi);
  return r;
}
template <>
__device__ __forceinline__ bf16x2_t make_pair<bf16x2_t>(float lo, float hi) {
  bf16x2_t r;
  r.x = static_cast<__bf16>(lo);
  r.y = static_cast<__bf16>(hi);
  return r;
}

constexpr uint32_t kI8Flip = 0x80808080u;    // two's complement -> offset binary
constexpr uint32_t kF16Filler = 0x64646464u; // high byte of fp16 1024.0 .. 1279.0
constexpr float kI8Offset = 1152.0f;         // 1024 + 128

// ---- K side: 16 raw bytes -> pairs along the head dimension -------------------------------
template <int KIND>
__device__ __forceinline__ void k_pairs(const uint4_t& r, typename KVTraits<KIND>::pair_t* out) {
  using P = typename KVTraits<KIND>::pair_t;
  if constexpr (KIND == KV_BF16 || KIND == KV_F16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t word = r[j];  // copy first: bit_cast straight from a vector-element lvalue reads element 0
      out[j] = __builtin_bit_cast(P, word);
    }
  } else if constexpr (KIND == KV_I8) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t u = r[j] ^ kI8Flip;
      out[2 * j] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, u, 0x04010400u));
      out[2 * j + 1] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, u, 0x04030402u));
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8(r[j], false);
      const float2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8(r[j], true);
      out[2 * j] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(lo.x, lo.y));
      out[2 * j + 1] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(hi.x, hi.y));
    }
  }
}

// ---- V side: two loads of the same lane (tokens t and t + TPL) -> pairs along the token axis
template <int KIND>
__device__ __forceinline__ void v_pairs(const uint4_t& a, const uint4_t& b, typename KVTraits<KIND>::pair_t* out) {
  using P = typename KVTraits<KIND>::pair_t;
  if constexpr (KIND == KV_BF16 || KIND == KV_F16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      out[2 * j] = __builtin_bit_cast(P, __builtin_amdgcn_perm(b[j], a[j], 0x05040100u));
      out[2 * j + 1] = __builtin_bit_cast(P, __builtin_amdgcn_perm(b[j], a[j], 0x07060302u));
    }
  } else if constexpr (KIND == KV_I8) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t ua = a[j] ^ kI8Flip, ub = b[j] ^ kI8Flip;
      const uint32_t x01 = __builtin_amdgcn_perm(ub, ua, 0x05010400u);  // a0 b0 a1 b1
      const uint32_t x23 = __builtin_amdgcn_perm(ub, ua, 0x07030602u);  // a2 b2 a3 b3
      out[4 * j + 0] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, x01, 0x04010400u));
      out[4 * j + 1] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, x01, 0x04030402u));
      out[4 * j + 2] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, x23, 0x04010400u));
      out[4 * j + 3] = __builtin_bit_cast(P, __builtin_amdgcn_perm(kF16Filler, x23, 0x04030402u));
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t x01 = __builtin_amdgcn_perm(b[j], a[j], 0x05010400u);
      const uint32_t x23 = __builtin_amdgcn_perm(b[j], a[j], 0x07030602u);
      const float2_t p0 = __builtin_amdgcn_cvt_pk_f32_fp8(x01, false);
      const float2_t p1 = __builtin_amdgcn_cvt_pk_f32_fp8(x01, true);
      const float2_t p2 = __builtin_amdgcn_cvt_pk_f32_fp8(x23, false);
      const float2_t p3 = __builtin_amdgcn_cvt_pk_f32_fp8(x23, true);
      out[4 * j + 0] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(p0.x, p0.y));
      out[4 * j + 1] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(p1.x, p1.y));
      out[4 * j + 2] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(p2.x, p2.y));
      out[4 * j + 3] = __builtin_bit_cast(P, __builtin_amdgcn_cvt_pkrtz(p3.x, p3.y));
    }
  }
}

__device__ __forceinline__ uint4_t load16(const void* base, int64_t byte_offset) {
  return *reinterpret_cast<const uint4_t*>(static_cast<const char*>(base) + byte_offset);
}

// first key the query may see (attention.cu:586-588): max(0, L_b - window_left) under a window, else 0
__device__ __forceinline__ int first_allowed_key(int length, int window_left) {
  if (window_left < 0) return 0;
  const int start = length - 1 - window_left;
  return start > 0 ? start : 0;
}

template <int KIND, int D, int G>
__global__ __launch_bounds__(kDecodeThreads) void decode_split_kernel(DecodeParams p) {
  using T = KVTraits<KIND>;
  using P = typename T::pair_t;
  constexpr int ES = T::kBytes;
  constexpr int EPL = 16 / ES;         // elements per lane per load
  constexpr int NP = EPL / 2;          // K pairs per lane per load
  constexpr int LPT = D / EPL;         // lanes per token row
  constexpr int TPL = kWave / LPT;     // token rows per load instruction
  constexpr int NL = TPL >= 16 ? 4 : 8; // loads per tile
  constexpr int TILE = NL * TPL;
  constexpr float kPScale = T::kQuant ? 256.0f : 1.0f;  // keeps p * v_scale in fp16's normal range
  static_assert(LPT >= 4 && LPT <= 16 && (NL % 2) == 0, "unsupported head_dim for this kernel");

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int hw_count = p.heads_per_wg;
  const int tw_count = 4 / hw_count;
  const int hw = wave % hw_count;
  const int ts = wave / hw_count;
  const int b = blockIdx.y;
  const int c = blockIdx.x;
  const int kvh = blockIdx.z * hw_count + hw;
  const int grp = lane / LPT;
  const int dc = lane % LPT;

  const int length = p.cache_seqlens[b] + 1;
  const int first_allowed = first_allowed_key(length, p.window_left);
  const int chunk_begin = c * p.chunk;
  const int chunk_lo = max(chunk_begin, first_allowed);
  const int chunk_hi = min(chunk_begin + p.chunk, length);
  if (chunk_lo >= chunk_hi) return;  // uniform over the workgroup

  const int slice = p.chunk / tw_count;
  const int w_begin = chunk_begin + ts * slice;
  const int w_lo = max(w_begin, chunk_lo);
  const int w_hi = min(w_begin + slice, chunk_hi);

  // ---- queries: G heads x this lane's EPL dims, as 16-bit pairs ----------------------------
  P qp[G][NP];
  float qbias[G];
  const int h0 = kvh * p.group;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float qsum = 0.0f;
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      float a = 0.0f, bb = 0.0f;
      if (g < p.group) {
        const int64_t idx = (static_cast<int64_t>(b) * p.q_heads + h0 + g) * D + dc * EPL + 2 * j;
        a = load_as_float(p.q, idx, p.q_dtype);
        bb = load_as_float(p.q, idx + 1, p.q_dtype);
      }
      qp[g][j] = make_pair<P>(a, bb);
      qsum += static_cast<float>(qp[g][j].x) + static_cast<float>(qp[g][j].y);
    }
    qbias[g] = KIND == KV_I8 ? -kI8Offset * qsum : 0.0f;
  }

  float m[G], l[G], psum[G];
  float acc[G][EPL];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegInf;
    l[g] = 0.0f;
    psum[g] = 0.0f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[g][e] = 0.0f;
  }

  const int32_t* table_row = p.block_table + static_cast<int64_t>(b) * p.max_blocks;
  const int64_t row_bytes = static_cast<int64_t>(D) * ES;

  for (int t0 = w_begin; t0 < w_hi; t0 += TILE) {
    if (t0 + TILE <= w_lo) continue;  // tile entirely left of the window
    uint4_t kraw[NL], vraw[NL];
    float kmul[NL], vmul[NL];
    bool valid[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int t = t0 + i * TPL + grp;
      valid[i] = t >= w_lo && t < w_hi;
      const int tc = min(max(t, w_lo), w_hi - 1);
      int col, slot;
      if (p.bs_shift >= 0) {
        col = tc >> p.bs_shift;
        slot = tc & (p.block_size - 1);
      } else {
        col = tc / p.block_size;
        slot = tc - col * p.block_size;
      }
      const int64_t blk = table_row[col];
      const int64_t row = (blk * p.block_size + slot) * p.kv_heads + kvh;
      kraw[i] = load16(p.k_cache, row * row_bytes + dc * 16);
      vraw[i] = load16(p.v_cache, row * row_bytes + dc * 16);
      if constexpr (T::kQuant) {
        kmul[i] = load_scale(p.k_scale, row, p.scale_dtype) * p.scale_log2e;
        vmul[i] = load_scale(p.v_scale, row, p.scale_dtype) * kPScale;
      } else {
        kmul[i] = p.scale_log2e;
        vmul[i] = kPScale;
      }
    }

    // ---- scores ------------------------------------------------------------------------------
    float s[NL][G];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      P kd[NP];
      k_pairs<KIND>(kraw[i], kd);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float a = qbias[g];
#pragma unroll
        for (int j = 0; j < NP; ++j) a = dot2(kd[j], qp[g][j], a);
#pragma unroll
        for (int mask = 1; mask < LPT; mask <<= 1) a += wave_xor(a, mask);
        s[i][g] = valid[i] ? a * kmul[i] : kNegInf;
      }
    }

    // ---- online softmax, per lane group --------------------------------------------------------
    float msafe[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mt = s[0][g];
#pragma unroll
      for (int i = 1; i < NL; ++i) mt = fmaxf(mt, s[i][g]);
      const float m_new = fmaxf(m[g], mt);
      msafe[g] = m_new == kNegInf ? 0.0f : m_new;
      const float alpha = fast_exp2(m[g] - msafe[g]);
      m[g] = m_new;
      l[g] *= alpha;
      psum[g] *= alpha;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][e] *= alpha;
    }

    // ---- P.V over token pairs --------------------------------------------------------------------
#pragma unroll
    for (int ip = 0; ip < NL / 2; ++ip) {
      P vp[EPL];
      v_pairs<KIND>(vraw[2 * ip], vraw[2 * ip + 1], vp);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float p0 = fast_exp2(s[2 * ip][g] - msafe[g]);
        const float p1 = fast_exp2(s[2 * ip + 1][g] - msafe[g]);
        l[g] += p0 + p1;
        const P pp = make_pair<P>(p0 * vmul[2 * ip], p1 * vmul[2 * ip + 1]);
        if constexpr (KIND == KV_I8) psum[g] += static_cast<float>(pp.x) + static_cast<float>(pp.y);
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = dot2(vp[e], pp, acc[g][e]);
      }
    }
  }

  // ---- merge the TPL lane-group states of this wave ----------------------------------------------
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mw = m[g];
#pragma unroll
    for (int mask = LPT; mask < kWave; mask <<= 1) mw = fmaxf(mw, wave_xor(mw, mask));
    const float ms = mw == kNegInf ? 0.0f : mw;
    const float f = fast_exp2(m[g] - ms);
    float lw = l[g] * f;
#pragma unroll
    for (int mask = LPT; mask < kWave; mask <<= 1) lw += wave_xor(lw, mask);
    const float off = KIND == KV_I8 ? kI8Offset * psum[g] : 0.0f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = (acc[g][e] - off) * (f * (1.0f / kPScale));
#pragma unroll
      for (int mask = LPT; mask < kWave; mask <<= 1) a += wave_xor(a, mask);
      acc[g][e] = a;
    }
    m[g] = mw;
    l[g] = lw;
  }

  // ---- merge the waves that share this KV head, write the chunk's partial ------------------------
  __shared__ float sm_acc[4][G][D];
  __shared__ float sm_ml[4][G][2];
  if (tw_count > 1) {
    if (grp == 0) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) sm_acc[wave][g][dc * EPL + e] = acc[g][e];
        if (dc == 0) {
          sm_ml[wave][g][0] = m[g];
          sm_ml[wave][g][1] = l[g];
        }
      }
    }
    __syncthreads();
    if (ts != 0) return;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mm = m[g];
      for (int w2 = 1; w2 < tw_count; ++w2) mm = fmaxf(mm, sm_ml[hw + w2 * hw_count][g][0]);
      const float ms = mm == kNegInf ? 0.0f : mm;
      const float f0 = fast_exp2(m[g] - ms);
      float ll = l[g] * f0;
#pragma unroll
      for (int e = 0; e < EPL; ++e) acc[g][e] *= f0;
      for (int w2 = 1; w2 < tw_count; ++w2) {
        const int ow = hw + w2 * hw_count;
        const float f = fast_exp2(sm_ml[ow][g][0] - ms);
        ll += sm_ml[ow][g][1] * f;
        if (grp == 0) {
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[g][e] += sm_acc[ow][g][dc * EPL + e] * f;
        }
      }
      m[g] = mm;
      l[g] = ll;
    }
  }

  if (grp == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g < p.group) {
        const int64_t prow = (static_cast<int64_t>(b) * p.q_heads + h0 + g) * p.max_parts + c;
        float* dst = p.part_acc + prow * D + dc * EPL;
#pragma unroll
        for (int e = 0; e < EPL; e += 4) {
          float4_t v4 = {acc[g][e], acc[g][e + 1], acc[g][e + 2], acc[g][e + 3]};
          *reinterpret_cast<float4_t*>(dst + e) = v4;
        }
        if (dc == 0) {
          p.part_ml[prow * 2] = m[g];
          p.part_ml[prow * 2 + 1] = l[g];
        }
      }
    }
  }
}

// Declared here, defined in one instantiation unit per KV kind (keeps compile times parallel).
typedef void (*decode_split_fn)(DecodeParams);
decode_split_fn decode_split_lookup_bf16(int head_dim, int group);
decode_split_fn decode_split_lookup_f16(int head_dim, int group);
decode_split_fn decode_split_lookup_i8(int head_dim, int group);
decode_split_fn decode_split_lookup_fp8(int head_dim, int group);

template <int KIND>
decode_split_fn decode_split_lookup_impl(int head_dim, int group) {
#define ARENO_PICK(DD, GG) \
  if (head_dim == DD && group <= GG) return decode_split_kernel<KIND, DD, GG>;
  ARENO_PICK(128, 1)
  ARENO_PICK(128, 2)
  ARENO_PICK(128, 4)
  ARENO_PICK(128, 7)
  ARENO_PICK(128, 8)
  ARENO_PICK(64, 1)
  ARENO_PICK(64, 2)
  ARENO_PICK(64, 4)
  ARENO_PICK(64, 8)
#undef ARENO_PICK
  return nullptr;
}

}  // namespace areno
