// Host launcher of the paged decode op plus its two small kernels:
//   decode_split_generic_kernel  -- any dtype / head_dim <= 512 / head ratio; one wave per (chunk, row)
//   decode_reduce_kernel         -- log-sum-exp merge of the chunk partials (attention.cu:656-702 in the
//                                   reference), normalise, cast to the query dtype
// The fast split kernels live in paged_decode_kernels.hpp.

#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "cache_row_quant.hpp"
#include "decode_mfma_kernels.hpp"

namespace areno {

int validate_paged_cache(const areno_paged_cache* c, const char* op);

namespace {

constexpr int kGenericMaxPerLane = 8;  // head_dim <= 512

__global__ __launch_bounds__(kWave) void decode_split_generic_kernel(DecodeParams p) {
  const int lane = threadIdx.x;
  const int row = blockIdx.x;
  const int c = blockIdx.y;
  const int b = row / p.q_heads;
  const int h = row - b * p.q_heads;
  const int kvh = h / p.group;
  const int d = p.head_dim;

  const int length = p.cache_seqlens[b] + 1;
  const int first_allowed = first_allowed_key(length, p.window_left);
  const int lo = max(c * p.chunk, first_allowed);
  const int hi = min((c + 1) * p.chunk, length);
  if (lo >= hi) return;

  float q[kGenericMaxPerLane], acc[kGenericMaxPerLane];
#pragma unroll
  for (int e = 0; e < kGenericMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    q[e] = idx < d ? load_as_float(p.q, static_cast<int64_t>(row) * d + idx, p.q_dtype) : 0.0f;
    acc[e] = 0.0f;
  }
  const bool quant = p.cache_dtype == ARENO_DT_I8 || p.cache_dtype == ARENO_DT_FP8_E4M3;
  float m = kNegInf, l = 0.0f;
  const int32_t* table_row = p.block_table + static_cast<int64_t>(b) * p.max_blocks;
  for (int t = lo; t < hi; ++t) {
    const int col = t / p.block_size;
    const int slot = t - col * p.block_size;
    const int64_t blk = table_row[col];
    const int64_t r = (blk * p.block_size + slot) * p.kv_heads + kvh;
    float dot = 0.0f;
    float v[kGenericMaxPerLane];
#pragma unroll
    for (int e = 0; e < kGenericMaxPerLane; ++e) {
      const int idx = lane + e * kWave;
      if (idx < d) {
        dot += q[e] * load_as_float(p.k_cache, r * d + idx, p.cache_dtype);
        v[e] = load_as_float(p.v_cache, r * d + idx, p.cache_dtype);
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
    const float alpha = fast_exp2(m - m_new);  // m = -inf on the first key -> 0
    const float beta = fast_exp2(s - m_new);
    l = l * alpha + beta;
    m = m_new;
    const float bv = beta * vs;
#pragma unroll
    for (int e = 0; e < kGenericMaxPerLane; ++e) acc[e] = acc[e] * alpha + bv * v[e];
  }
  const int64_t prow = static_cast<int64_t>(row) * p.max_parts + c;
#pragma unroll
  for (int e = 0; e < kGenericMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    if (idx < d) p.part_acc[prow * d + idx] = acc[e];
  }
  if (lane == 0) {
    p.part_ml[prow * 2] = m;
    p.part_ml[prow * 2 + 1] = l;
  }
}

constexpr int kReduceRows = 4;

__global__ __launch_bounds__(kReduceRows* kWave) void decode_reduce_kernel(DecodeParams p) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = blockIdx.x * kReduceRows + (threadIdx.x >> 6);
  if (row >= p.batch * p.q_heads) return;
  const int b = row / p.q_heads;
  const int d = p.head_dim;
  const int length = p.cache_seqlens[b] + 1;
  const int first_allowed = first_allowed_key(length, p.window_left);
  const int c_lo = first_allowed / p.chunk;
  const int c_hi = (length - 1) / p.chunk;

  float acc[kGenericMaxPerLane];
#pragma unroll
  for (int e = 0; e < kGenericMaxPerLane; ++e) acc[e] = 0.0f;
  float m = kNegInf, l = 0.0f;
  const int64_t base = static_cast<int64_t>(row) * p.max_parts;
  for (int c = c_lo; c <= c_hi && c < p.max_parts; ++c) {
    const float part_m = p.part_ml[(base + c) * 2];
    const float part_l = p.part_ml[(base + c) * 2 + 1];
    if (part_l == 0.0f) continue;  // a partial without keys contributes nothing (attention.cu:680-682)
    const float m_new = fmaxf(m, part_m);
    const float alpha = fast_exp2(m - m_new);
    const float beta = fast_exp2(part_m - m_new);
    const float* part = p.part_acc + (base + c) * d;
#pragma unroll
    for (int e = 0; e < kGenericMaxPerLane; ++e) {
      const int idx = lane + e * kWave;
      if (idx < d) acc[e] = acc[e] * alpha + part[idx] * beta;
    }
    l = l * alpha + part_l * beta;
    m = m_new;
  }
#pragma unroll
  for (int e = 0; e < kGenericMaxPerLane; ++e) {
    const int idx = lane + e * kWave;
    if (idx < d) store_from_float(p.out, static_cast<int64_t>(row) * d + idx, p.q_dtype, acc[e] / l);
  }
}

// Merge of the MFMA path's partials.  The units that own quanta of an item wrote one partial each: a per-row item
// into slot (unit + row) of the per-row region, a shared-prefix item (grouped mode) into slot (unit + item) of the
// shared region, where the row's head sits in column (row - first row) * G + head of its kv head.  One wave per
// (row, q head) gathers the candidates of both kinds, kMergeChunk at a time, and merges them with the log-sum-exp
// recurrence of the reference's reduce kernel (areno/accel/csrc/attention.cu:656-702).
//
// The token being appended (items.append_in_merge): the streaming waves of the split kernel read only what is in the
// pages, and this kernel, which owns the (row, head) anyway, does what the reference's update kernel
// (areno/accel/csrc/attention.cu:526-553) and the last key of its split kernel do: the wave reads the row of
// k_update / v_update of its kv head, quantizes it with the cache writer's closed form, the wave of the kv head's
// first q head stores codes and scale at (block_table[b, L / bs], L % bs) -- skipped, like the cache writer does, when
// the column or the page id lies outside the table or the pool -- and the token enters the merge as a partial of its
// own with m = q . k_new, l = 1, acc = v_new, both as a reader of the page would see them.
//
// Memory round trips, which are what this kernel's time is made of: (1) the row's entry of the plan (or the prefix
// sums its units follow from), its length and the q / k_update / v_update rows; (2) the append's block id and, for up
// to kMergeChunk candidates at once, (m, l) and the accumulator row together -- a candidate's row is fetched before
// its weight is known; (3) the stores.
constexpr int kMergeChunk = 8;

// The arguments in front of the parameter block are what the kernel's first loads are addressed with: as leading
// scalar arguments they reach the wave in registers at its start (kernel-argument preload, at most 16 words), while
// the block behind them takes a fetch of its own.
//
// The kernel's time is those round trips plus what a wave issues in between, and with seven waves on a CU nothing
// hides a wave's own instructions, so the kernel is instantiated for what would otherwise be decided at run time --
// the query dtype (QDT), the cache dtype (CDT: QDT itself for 16-bit pages, ARENO_DT_I8, ARENO_DT_FP8_E4M3), whether
// a plan brings the row's unit ranges (PLANNED) -- and its index arithmetic avoids divisions: the grid is (q heads /
// kReduceRows, rows), the kv head of a q head and the page column of a position are multiplications by constants the
// launcher derives; candidates of a kind sit a constant stride apart, so their addresses are a base plus a multiple.
// Against a kernel that decided all of this at run time: a fifth of the instructions, 5.6 instead of 7.6 us per launch
// at batch 64.

// Candidates of one round trip: (m, l) and the lane's elements of the accumulator row.
template <int N, int EPW>
struct MergeChunk {
  static constexpr int kSize = N;
  float m[N], l[N];
  float v[N][EPW];
};

// The kernel keeps to few registers (48 at head dim 128): a variant that fetched 32 candidates per round trip for rows
// with many of them took 160 and every launch of it twice as long, whether or not a row had that many.  Rows with many
// candidates -- a small batch spreads each row over all units: 256 candidates at batch 1 -- are served by more waves
// instead: MW waves share a (row, head), wave w takes the chunks w, w + MW, ..., and wave 0 combines their results
// through LDS (MW = 1: a workgroup of kReduceRows waves takes that many heads of a row, no LDS).  The launcher picks
// MW from the batch size and the number of units, which is all it knows of the lengths.
template <int EPW, int QDT, int CDT, bool PLANNED, int MW>  // EPW: head-dimension elements per lane, head_dim <= 64 EPW
__global__ __launch_bounds__((MW == 1 ? kReduceRows : MW) * kWave) void decode_reduce_slots_kernel(
    const int32_t* plan_rows, const int32_t* cache_seqlens, const void* q_rows, const void* k_update,
    const void* v_update, int32_t q_heads, int32_t kv_heads, int32_t group, uint32_t group_magic, int32_t head_dim,
    MfmaDecodeParams mp) {
  const DecodeParams& p = mp.d;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // (in a scalar register)
  const int b = blockIdx.y;
  const int h = MW == 1 ? blockIdx.x * kReduceRows + wave : blockIdx.x;
  const int part = MW == 1 ? 0 : wave;  // which share of the row's candidates this wave merges
  if (h >= q_heads) return;
  const int row = b * q_heads + h;
  const int kvh = group == 1 ? h : static_cast<int>(__umulhi(static_cast<uint32_t>(h), group_magic));  // h / group
  const int d = head_dim;
  const ItemShape& shape = mp.items;
  // (the launcher passes the update rows only when this launch folds them in; of the waves that share a row, the first
  // one takes the new token)
  const bool append = k_update != nullptr && part == 0;

  // ---- round trip 1 ---------------------------------------------------------------------------------------------------
  // units that hold partials of the row: its own item's and, with prefix groups, its sub-group's shared item's
  int own_lo = 0, own_n = 0, sh_lo = 0, sh_n = 0, sh_item = 0, sh_col = 0;
  int4_t planned_units = {0, 0, 0, 0};
  int cum_total = 0, cum_own = 0, cum_own_end = 0, cum_sh = 0, cum_sh_end = 0;
  if (shape.num_shared > 0) {
    const int gi = b / shape.group_rows;
    const int j = (b - gi * shape.group_rows) / shape.cols_seqs;
    sh_item = gi * shape.subs_per_group + j;
    const int first_row = gi * shape.group_rows + j * shape.cols_seqs;
    sh_col = kvh * 16 + (b - first_row) * group + (h - kvh * group);
  }
  if constexpr (PLANNED) {
    planned_units = *reinterpret_cast<const int4_t*>(plan_rows + 4 * static_cast<int64_t>(b));
    cum_total = plan_rows[-4];
  } else {
    const int32_t* cum = mp.cum_out;
    const int v_own = shape.num_shared + b;
    cum_total = cum[shape.num_items()];
    cum_own = cum[v_own];
    cum_own_end = cum[v_own + 1];
    cum_sh = cum[sh_item];  // (entry 0 and 1 when there are no shared items: read and not used)
    cum_sh_end = cum[sh_item + 1];
  }
  // the update rows and the query row (stand-ins from the query tensor when nothing is appended: read, not used)
  uint16_t qraw[EPW], kraw[EPW], vraw[EPW];
  const int pos = cache_seqlens[b];
  {
    const uint16_t* ksrc = static_cast<const uint16_t*>(append ? k_update : q_rows);
    const uint16_t* vsrc = static_cast<const uint16_t*>(append ? v_update : q_rows);
    const int64_t src_base = (static_cast<int64_t>(b) * kv_heads + kvh) * d;
    const int64_t q_base = static_cast<int64_t>(row) * d;
#pragma unroll
    for (int e = 0; e < EPW; ++e) {
      const int idx = min(lane + e * kWave, d - 1);
      kraw[e] = ksrc[src_base + idx];
      vraw[e] = vsrc[src_base + idx];
      qraw[e] = static_cast<const uint16_t*>(q_rows)[q_base + idx];
    }
  }
  auto widen = [](uint16_t raw) { return QDT == ARENO_DT_BF16 ? bf16_bits_to_float(raw) : f16_bits_to_float(raw); };
  if constexpr (PLANNED) {
    own_lo = planned_units[0];
    own_n = planned_units[1];
    sh_lo = planned_units[2];
    sh_n = planned_units[3];
  } else {
    const UnitGeometry geo = make_unit_geometry(cum_total, mp.num_units);
    if (cum_own_end > cum_own) {
      int last;
      item_units(geo, shape.switch_quanta, cum_own, cum_own_end, own_lo, last);
      own_n = last - own_lo + 1;
    }
    if (shape.num_shared > 0 && cum_sh_end > cum_sh) {
      int last;
      item_units(geo, shape.switch_quanta, cum_sh, cum_sh_end, sh_lo, last);
      sh_n = last - sh_lo + 1;
    }
  }
  const int total = own_n + sh_n;

  // ---- round trip 2: the page the new token goes to, and the candidates ------------------------------------------------
  // position -> (block-table column, slot) by the launcher's multiply-shift constants (any page size); the id of a
  // clamped column is read whatever the position and dropped when the position has no column
  const int col = static_cast<int>(__umulhi(static_cast<uint32_t>(max(pos, 0)), mp.bs_magic) >> mp.bs_post);
  const int slot = pos - col * p.block_size;
  const int blk = p.block_table[static_cast<int64_t>(b) * p.max_blocks + min(col, p.max_blocks - 1)];
  // Candidate c of the row is the partial of unit own_lo + c (c < own_n), then of unit sh_lo + c - own_n of the shared
  // item: consecutive candidates of a kind sit a constant stride apart, so an address is a base plus a multiple.  A
  // candidate past the row's last one reads the last one again (a line this wave fetches anyway) and is masked out;
  // a row without candidates reads slot b of the per-row region, which nothing writes, and masks it out.
  const int64_t own_row0 = static_cast<int64_t>(own_lo + b) * q_heads + h;
  const int64_t sh_row0 = static_cast<int64_t>(sh_lo + sh_item) * kv_heads * 16 + sh_col;
  const int64_t sh_row_stride = static_cast<int64_t>(kv_heads) * 16;
  const float* const sh_ml = sh_n > 0 ? mp.shared_ml : p.part_ml;  // (never dereferenced without shared candidates)
  const float* const sh_acc = sh_n > 0 ? mp.shared_acc : p.part_acc;
  auto load_chunk = [&](int base, auto& ch) {
    constexpr int N = std::remove_reference_t<decltype(ch)>::kSize;
    float2_t pair[N];
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const int c = max(min(base + j, total - 1), 0);
      const bool own = c < own_n || total == 0;
      const int64_t prow = own ? own_row0 + static_cast<int64_t>(c) * q_heads : sh_row0 + (c - own_n) * sh_row_stride;
      const float* ml = (own ? p.part_ml : sh_ml) + prow * 2;
      const float* part = (own ? p.part_acc : sh_acc) + prow * d;
      pair[j] = float2_t{kNegInf, 0.0f};
#pragma unroll
      for (int e = 0; e < EPW; ++e) ch.v[j][e] = 0.0f;
      if (base + j < total) {
        pair[j] = *reinterpret_cast<const float2_t*>(ml);
#pragma unroll
        for (int e = 0; e < EPW; ++e) ch.v[j][e] = part[min(lane + e * kWave, d - 1)];
      }
    }
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const bool present = base + j < total;  // (every unit of a row's range holds quanta of the row)
      // a partial without keys contributes nothing (attention.cu:680-682 in the reference)
      ch.m[j] = (present && pair[j][1] != 0.0f) ? pair[j][0] : kNegInf;
      ch.l[j] = present ? pair[j][1] : 0.0f;
#pragma unroll
      for (int e = 0; e < EPW; ++e) ch.v[j][e] = (present && lane + e * kWave < d) ? ch.v[j][e] : 0.0f;
    }
  };
  MergeChunk<kMergeChunk, EPW> first;
  load_chunk(part * kMergeChunk, first);

  // ---- the new token: quantize, store, m = q . k_new, l = 1, acc = v_new ----------------------------------------------
  float acc[EPW];
#pragma unroll
  for (int e = 0; e < EPW; ++e) acc[e] = 0.0f;
  float m = kNegInf, l = 0.0f;
  if (append) {
    const bool ok = pos >= 0 && col < p.max_blocks && blk >= 0 && blk < mp.num_blocks;
    const bool store = ok && mp.write_append != 0 && h == kvh * group;
    const int64_t dst_row = (static_cast<int64_t>(ok ? blk : 0) * p.block_size + slot) * kv_heads + kvh;
    float kx[EPW], vx[EPW], qv[EPW];
#pragma unroll
    for (int e = 0; e < EPW; ++e) {
      const bool in = lane + e * kWave < d;
      kx[e] = in ? widen(kraw[e]) : 0.0f;
      vx[e] = in ? widen(vraw[e]) : 0.0f;
      qv[e] = in ? widen(qraw[e]) : 0.0f;
    }
    float khat[EPW], vhat[EPW];
    if constexpr (CDT == ARENO_DT_I8 || CDT == ARENO_DT_FP8_E4M3) {
      quantize_row<EPW>(kx, lane, d, dst_row, const_cast<void*>(p.k_cache), const_cast<void*>(p.k_scale), CDT,
                        p.scale_dtype, store, khat);
      quantize_row<EPW>(vx, lane, d, dst_row, const_cast<void*>(p.v_cache), const_cast<void*>(p.v_scale), CDT,
                        p.scale_dtype, store, vhat);
    } else {
      // 16-bit pages of the query's dtype hold the update row as it is
#pragma unroll
      for (int e = 0; e < EPW; ++e) {
        const int idx = lane + e * kWave;
        if (store && idx < d) {
          static_cast<uint16_t*>(const_cast<void*>(p.k_cache))[dst_row * d + idx] = kraw[e];
          static_cast<uint16_t*>(const_cast<void*>(p.v_cache))[dst_row * d + idx] = vraw[e];
        }
        khat[e] = kx[e];
        vhat[e] = vx[e];
      }
    }
    float dot = 0.0f;
#pragma unroll
    for (int e = 0; e < EPW; ++e) dot += qv[e] * khat[e];
    m = wave_sum_fast(dot) * p.scale_log2e;
    l = 1.0f;
#pragma unroll
    for (int e = 0; e < EPW; ++e) acc[e] = vhat[e];
  }

  // ---- merge ----------------------------------------------------------------------------------------------------------
  auto merge_chunk = [&](const auto& ch) {
    constexpr int N = std::remove_reference_t<decltype(ch)>::kSize;
    float m_new = m;
#pragma unroll
    for (int j = 0; j < N; ++j) m_new = fmaxf(m_new, ch.m[j]);
    const float m_safe = m_new == kNegInf ? 0.0f : m_new;
    const float alpha = fast_exp2(m - m_safe);
    l *= alpha;
#pragma unroll
    for (int e = 0; e < EPW; ++e) acc[e] *= alpha;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float w = fast_exp2(ch.m[j] - m_safe);  // 0 for absent candidates
      l += w * ch.l[j];
#pragma unroll
      for (int e = 0; e < EPW; ++e) acc[e] += w * ch.v[j][e];
    }
    m = m_new;
  };
  merge_chunk(first);
  for (int base = (part + MW) * kMergeChunk; base < total; base += MW * kMergeChunk) {
    MergeChunk<kMergeChunk, EPW> more;
    load_chunk(base, more);
    merge_chunk(more);
  }
  if constexpr (MW > 1) {
    // the waves' (m, l, acc) meet in LDS; wave 0 combines them in wave order and writes the row
    __shared__ float s_ml[MW][2];
    __shared__ float s_acc[MW][EPW * kWave];
    if (lane == 0) {
      s_ml[part][0] = m;
      s_ml[part][1] = l;
    }
#pragma unroll
    for (int e = 0; e < EPW; ++e) s_acc[part][lane + e * kWave] = acc[e];
    __syncthreads();
    if (part != 0) return;
    float m_all = kNegInf;
#pragma unroll
    for (int w2 = 0; w2 < MW; ++w2) m_all = fmaxf(m_all, s_ml[w2][0]);
    const float m_safe = m_all == kNegInf ? 0.0f : m_all;
    l = 0.0f;
#pragma unroll
    for (int e = 0; e < EPW; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < MW; ++w2) {
      const float wgt = fast_exp2(s_ml[w2][0] - m_safe);  // 0 for a wave without candidates
      l += wgt * s_ml[w2][1];
#pragma unroll
      for (int e = 0; e < EPW; ++e) acc[e] += wgt * s_acc[w2][lane + e * kWave];
    }
  }
#pragma unroll
  for (int e = 0; e < EPW; ++e) {
    const int idx = lane + e * kWave;
    if (idx < d) store_from_float(p.out, static_cast<int64_t>(row) * d + idx, QDT, acc[e] / l);
  }
}

typedef void (*reduce_slots_fn)(const int32_t*, const int32_t*, const void*, const void*, const void*, int32_t, int32_t,
                                int32_t, uint32_t, int32_t, MfmaDecodeParams);
// the narrowest instantiation that covers the head: the kernel is a few hundred instructions per wave and mostly
// launch latency, so slots that would only be predicated off are worth leaving out
template <int QDT, int CDT, bool PLANNED, int MW>
reduce_slots_fn reduce_slots_kernel_by_width(int head_dim) {
  if (head_dim <= 64) return decode_reduce_slots_kernel<1, QDT, CDT, PLANNED, MW>;
  if (head_dim <= 128) return decode_reduce_slots_kernel<2, QDT, CDT, PLANNED, MW>;
  if (head_dim <= 256) return decode_reduce_slots_kernel<4, QDT, CDT, PLANNED, MW>;
  return decode_reduce_slots_kernel<kGenericMaxPerLane, QDT, CDT, PLANNED, MW>;
}
template <int QDT, int CDT, bool PLANNED>
reduce_slots_fn reduce_slots_kernel_by_waves(int head_dim, int waves) {
  if (waves == 1) return reduce_slots_kernel_by_width<QDT, CDT, PLANNED, 1>(head_dim);
  if (waves == 4) return reduce_slots_kernel_by_width<QDT, CDT, PLANNED, 4>(head_dim);
  return reduce_slots_kernel_by_width<QDT, CDT, PLANNED, 16>(head_dim);
}
template <int QDT, bool PLANNED>
reduce_slots_fn reduce_slots_kernel_by_cache(int head_dim, int cache_dtype, int waves) {
  if (cache_dtype == ARENO_DT_I8) return reduce_slots_kernel_by_waves<QDT, ARENO_DT_I8, PLANNED>(head_dim, waves);
  if (cache_dtype == ARENO_DT_FP8_E4M3) return reduce_slots_kernel_by_waves<QDT, ARENO_DT_FP8_E4M3, PLANNED>(head_dim, waves);
  return reduce_slots_kernel_by_waves<QDT, QDT, PLANNED>(head_dim, waves);  // 16-bit pages (an append needs them in q's dtype)
}
reduce_slots_fn reduce_slots_kernel_for(int head_dim, int q_dtype, int cache_dtype, bool planned, int waves) {
  if (q_dtype == ARENO_DT_BF16)
    return planned ? reduce_slots_kernel_by_cache<ARENO_DT_BF16, true>(head_dim, cache_dtype, waves)
                   : reduce_slots_kernel_by_cache<ARENO_DT_BF16, false>(head_dim, cache_dtype, waves);
  return planned ? reduce_slots_kernel_by_cache<ARENO_DT_F16, true>(head_dim, cache_dtype, waves)
                 : reduce_slots_kernel_by_cache<ARENO_DT_F16, false>(head_dim, cache_dtype, waves);
}
// Waves that share a (row, head) in the merge launch: a row has about units / batch + 2 candidates (the launcher knows
// no lengths; a long row among short ones has more), and a wave takes kMergeChunk of them per round trip.
int merge_waves_for(int units, int batch) {
  const int chunks = (units / (batch > 0 ? batch : 1) + 2 + kMergeChunk - 1) / kMergeChunk;
  return chunks <= 1 ? 1 : (chunks <= 4 ? 4 : 16);
}

// ---- geometry of the MFMA path ----------------------------------------------------------------------
constexpr int kMfmaWaves = ARENO_MFMA_NW;  // waves per workgroup
constexpr int kComputeUnits = 256;
// One workgroup per CU: a wave keeps one 32-token tile (K and V) in flight, and 1024 waves with a tile each already
// saturate the memory system; a second resident workgroup per CU only lengthens its queues and spreads the waves'
// finish times (measured, split kernel / whole step: bf16 pages, 16 KB tiles, 61.7 / 69.7 us with 512 workgroups
// against 59.1 / 65.8 us with 256; fp8 rollout 212.3 / 228.9 against 206.8 / 223.6; int8, 8 KB tiles, 32.9 / 41.6
// against 33.2 / 40.5: the split kernel's loss is made up by the merge, which has half the partials to read).
constexpr int kMfmaWorkgroups = kComputeUnits;
constexpr int kMfmaMaxUnits = kMfmaWorkgroups * kMfmaWaves;  // one kv head, every wave a unit of its own

// partials of `slots` slots, and behind them the dump row of the lanes that own no partial row
size_t mfma_partial_bytes(size_t slots, int q_heads, int head_dim) {
  const size_t bytes = (slots * q_heads * (static_cast<size_t>(head_dim) + 2) + kDecodeDumpFloats) * sizeof(float);
  return (bytes + 255) / 256 * 256;
}

size_t mfma_workspace_bytes(int batch, int q_heads, int head_dim) {
  const size_t slots = static_cast<size_t>(kMfmaMaxUnits) + batch;
  const size_t plan_words = (static_cast<size_t>(batch) + 1 + 63) / 64 * 64;
  return mfma_partial_bytes(slots, q_heads, head_dim) + plan_words * sizeof(int32_t);
}

// "valu" forces the vector-ALU split kernel (a diagnosis switch), anything else prefers the matrix-core kernel.
// Per-wave timestamps of the split kernel; set through areno_hip_debug_set_trace in ARENO_TRACE builds only.
unsigned long long* g_trace_buffer = nullptr;

bool prefer_mfma() {
  static const int choice = [] {
    const char* v = getenv("ARENO_DECODE_KERNEL");
    return (v != nullptr && strcmp(v, "valu") == 0) ? 0 : 1;
  }();
  return choice == 1;
}

struct Chunking {
  int chunk;
  int max_parts;
};

constexpr int kChunkQuantum = 256;  // multiple of every tile size times the largest token split
constexpr int kMaxParts = 64;

bool pick_chunking(int64_t block_size, int64_t max_blocks, int num_splits, Chunking* out) {
  const int64_t max_tokens = block_size * max_blocks;
  if (max_tokens <= 0 || max_tokens > 0x3fffffffLL) return false;
  int64_t chunk = kChunkQuantum;
  if (num_splits == 1) {
    chunk = (max_tokens + kChunkQuantum - 1) / kChunkQuantum * kChunkQuantum;
  } else {
    while ((max_tokens + chunk - 1) / chunk > kMaxParts) chunk *= 2;
  }
  out->chunk = static_cast<int>(chunk);
  out->max_parts = static_cast<int>((max_tokens + chunk - 1) / chunk);
  return true;
}

int log2_exact(int x) {
  if (x <= 0 || (x & (x - 1)) != 0) return -1;
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}

}  // namespace
}  // namespace areno

extern "C" size_t areno_hip_paged_decode_workspace_bytes(int32_t batch, int32_t q_heads, int32_t head_dim,
                                                         int32_t block_size, int32_t max_blocks, int32_t num_splits) {
  areno::Chunking ch;
  if (batch <= 0 || q_heads <= 0 || head_dim <= 0 || num_splits < 1) return 0;
  if (!areno::pick_chunking(block_size, max_blocks, num_splits, &ch)) return 0;
  const size_t rows = static_cast<size_t>(batch) * q_heads * ch.max_parts;
  size_t bytes = rows * (static_cast<size_t>(head_dim) + 2) * sizeof(float);
  bytes = (bytes + 255) / 256 * 256;
  const size_t mfma = areno::mfma_workspace_bytes(batch, q_heads, head_dim);
  return bytes > mfma ? bytes : mfma;
}

extern "C" int areno_hip_paged_decode(const areno_paged_cache* cache, const void* q, const void* k_update,
                                      const void* v_update, void* out, int32_t q_dtype, int32_t batch,
                                      int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                      const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                                      float softmax_scale, void* workspace, size_t workspace_bytes, void* stream) {
  return areno_hip_paged_decode_stages(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table,
                                       max_blocks, cache_seqlens, window_left, num_splits, softmax_scale, workspace,
                                       workspace_bytes, ARENO_STAGE_ALL, stream);
}

namespace areno {
namespace {

// Units (one per wave) the split kernel uses for a kv-head count and head dim: what the partial regions are indexed by.
struct MfmaGrid {
  int waves, head_split, heads_per_wg, head_groups, tok_splits, workgroups, units;
};
MfmaGrid mfma_grid_for(int kv_heads, int head_dim) {
  MfmaGrid g;
  g.waves = decode_mfma_waves(head_dim);
  g.head_split = decode_mfma_head_split(head_dim);
  const int heads = g.waves / g.head_split;  // kv heads a workgroup can serve at once
  g.heads_per_wg = (heads >= 4 && kv_heads % 4 == 0) ? 4 : ((heads >= 2 && kv_heads % 2 == 0) ? 2 : 1);
  g.head_groups = kv_heads / g.heads_per_wg;
  g.tok_splits = heads / g.heads_per_wg;
  g.workgroups = kMfmaWorkgroups / g.head_groups > 0 ? kMfmaWorkgroups / g.head_groups : 1;
  g.units = g.workgroups * g.tok_splits;
  return g;
}

// cum entries of the grouped item list (up to one shared item per row on top of the rows), kept 256-byte granular
size_t grouped_plan_bytes(int batch) { return ((2 * static_cast<size_t>(batch) + 64) * sizeof(int32_t) + 255) / 256 * 256; }

size_t shared_region_bytes(int kv_heads, int head_dim, int num_shared) {
  const size_t slots = static_cast<size_t>(mfma_grid_for(kv_heads, head_dim).units) + num_shared;
  return slots * kv_heads * 16 * (static_cast<size_t>(head_dim) + 2) * sizeof(float);
}

decode_mfma_fn mfma_lookup(const areno_paged_cache* cache, bool grouped) {
  const bool s16 = cache->scale_dtype == ARENO_DT_F16;
  switch (cache->cache_dtype) {
    case ARENO_DT_BF16: return decode_mfma_lookup_bf16(cache->head_dim, s16, grouped);
    case ARENO_DT_F16: return decode_mfma_lookup_f16(cache->head_dim, s16, grouped);
    case ARENO_DT_I8: return decode_mfma_lookup_i8(cache->head_dim, s16, grouped);
    case ARENO_DT_FP8_E4M3: return decode_mfma_lookup_fp8(cache->head_dim, s16, grouped);
    default: return nullptr;
  }
}

// Whether (and how) the matrix-core kernel serves a call: 16-bit or 8-bit caches, head_dim 64 / 128 / 192 / 256 / 512,
// up to 16 * kMaxHeadParts q heads per kv head (16 per column tile; further tiles of a kv head run as heads of their
// own that read the same pages), pages of at least 4 tokens, at most kMfmaMaxBatch rows.  Shared by the decode
// launcher and the plan builder, which must agree on the item list and the units.
constexpr int kMaxHeadParts = 8;

struct MfmaChoice {
  decode_mfma_fn fn;  // NULL: another kernel takes the call
  MfmaGrid grid;
  ItemShape items;
  int tile_tokens;
  int head_parts;  // column tiles per kv head
};
MfmaChoice choose_mfma(const areno_paged_cache* cache, int q_dtype, int batch, int q_heads, int window_left,
                       bool with_update, int group_rows, bool has_shared_lens) {
  MfmaChoice c;
  c.fn = nullptr;
  const int group = q_heads / cache->kv_heads;
  c.head_parts = (group + 15) / 16;
  c.grid = mfma_grid_for(cache->kv_heads * c.head_parts, cache->head_dim);
  // what changing items costs a wave, in 16-token quanta of streaming (measured: ~1.4 us against ~1.4 us per 32-token
  // tile of 8-bit pages, ~2.6 us per tile of 16-bit pages)
  c.items = ItemShape{batch, window_left, 0, is_quantized(cache->cache_dtype) ? 3 : 1, 0, 1, 1, 1};
  c.tile_tokens = decode_tile_tokens(is_quantized(cache->cache_dtype));
  const bool aligned = (reinterpret_cast<uintptr_t>(cache->k) % 16 == 0) && (reinterpret_cast<uintptr_t>(cache->v) % 16 == 0);
  // the kernel indexes cache rows (block, slot, head) with 32 bits
  const bool rows_fit = static_cast<double>(cache->num_blocks) * cache->block_size * cache->kv_heads < 4294967296.0;
  PageDivision division;
  if (!aligned || q_dtype == ARENO_DT_F32 || !prefer_mfma() || c.head_parts > kMaxHeadParts || batch > kMfmaMaxBatch || !rows_fit ||
      q_heads > 65535 ||
      !page_division(cache->block_size, &division))
    return c;
  // prefix groups: only without a window, when at least two rows fit side by side
  int cols_seqs = 0, subs_per_group = 0, num_shared = 0;
  if (has_shared_lens && window_left < 0) num_shared = shared_items_for(batch, group, group_rows, &cols_seqs, &subs_per_group);
  c.fn = mfma_lookup(cache, num_shared > 0);
  if (c.fn == nullptr && num_shared > 0) {
    // no grouped kernel for this shape: the plain matrix-core kernel, every row reading its own pages
    num_shared = 0;
    c.fn = mfma_lookup(cache, false);
  }
  if (c.fn == nullptr) return c;
  // The token being appended is folded in by the merge launch when its row can go into the page as it is (16-bit
  // pages of the query's dtype) or through the quantizer (8-bit pages); the streaming waves then read the cached
  // tokens only.
  c.items.append_in_merge = (with_update && (is_quantized(cache->cache_dtype) || q_dtype == cache->cache_dtype)) ? 1 : 0;
  if (num_shared > 0) {
    c.items.num_shared = num_shared;
    c.items.group_rows = group_rows;
    c.items.cols_seqs = cols_seqs;
    c.items.subs_per_group = subs_per_group;
  }
  return c;
}

// ---- the plan: item table, prefix sums and one record per unit, built once for all layers of a decode step ----------
struct PlanParams {
  const int32_t* cache_seqlens;
  const int32_t* shared_lens;
  const int32_t* block_table;
  int32_t* cum;
  int32_t* items;
  int32_t* units;
  int32_t* rows;
  ItemShape shape;
  int32_t num_units;
  int32_t block_size;
  int32_t max_blocks;
};

struct GlobalLens {
  const int32_t* len;
  const int32_t* glen;
  __device__ int row_len(int b) const { return len[b]; }
  __device__ int group_len(int g) const { return glen[g]; }
};
struct PlainItemTable {
  const int4_t* item;
  const int* cum_;
  __device__ ItemInfo info(int b) const {
    const int4_t r = item[b];
    return ItemInfo{r[0], r[1], r[2], r[3]};
  }
  __device__ int cum(int i) const { return cum_[i]; }
};

constexpr int kPlanThreads = 1024;

template <bool GROUPED>
__global__ __launch_bounds__(kPlanThreads) void decode_plan_kernel(PlanParams pp) {
  constexpr int kMaxItems = (GROUPED ? 2 : 1) * kMfmaMaxBatch;
  constexpr int SPT = kMaxItems / kPlanThreads;
  constexpr int kWaves = kPlanThreads / kWave;
  __shared__ __attribute__((aligned(16))) int4_t s_item[kMaxItems];
  __shared__ int s_cum[kMaxItems + 1];
  __shared__ int s_wave_tot[kWaves];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const ItemShape& shape = pp.shape;
  const int num_items = shape.num_items();
  const GlobalLens lens = {pp.cache_seqlens, pp.shared_lens};
  int nt[SPT];
  int local = 0;
#pragma unroll
  for (int j = 0; j < SPT; ++j) {
    const int v = SPT * tid + j;
    nt[j] = 0;
    if (v < num_items) {
      const ItemInfo it = item_info<GROUPED>(shape, lens, v);
      const int4_t r = {it.lo, it.end, it.row, it.nseq};
      s_item[v] = r;
      *reinterpret_cast<int4_t*>(pp.items + 4 * static_cast<int64_t>(v)) = r;
      nt[j] = it.extent(shape.switch_quanta);
    }
    local += nt[j];
  }
  int incl = local;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int v = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += v;
  }
  if (lane == kWave - 1) s_wave_tot[wave] = incl;
  __syncthreads();
  int excl = incl - local;
  for (int w2 = 0; w2 < wave; ++w2) excl += s_wave_tot[w2];
#pragma unroll
  for (int j = 0; j < SPT; ++j) {
    const int v = SPT * tid + j;
    if (v <= num_items) {
      s_cum[v] = excl;
      pp.cum[v] = excl;
    }
    excl += nt[j];
  }
  if (tid == kPlanThreads - 1 && SPT * (tid + 1) <= num_items) {
    s_cum[SPT * (tid + 1)] = excl;
    pp.cum[SPT * (tid + 1)] = excl;
  }
  __syncthreads();
  const PlainItemTable table = {s_item, s_cum};
  const UnitGeometry geo = make_unit_geometry(s_cum[num_items], pp.num_units);
  // per row, for the merge kernel: first unit and number of units of its own item and of its sub-group's shared item;
  // in front of the rows the total of the cost line
  if (tid == 0) *reinterpret_cast<int4_t*>(pp.rows - 4) = int4_t{s_cum[num_items], 0, 0, 0};
  for (int b = tid; b < shape.batch; b += kPlanThreads) {
    int4_t r = {0, 0, 0, 0};
    const int v_own = shape.num_shared + b;
    if (s_cum[v_own + 1] > s_cum[v_own]) {
      int first, last;
      item_units(geo, shape.switch_quanta, s_cum[v_own], s_cum[v_own + 1], first, last);
      r[0] = first;
      r[1] = last - first + 1;
    }
    if (GROUPED) {
      const int gi = b / shape.group_rows;
      const int sh_item = gi * shape.subs_per_group + (b - gi * shape.group_rows) / shape.cols_seqs;
      if (s_cum[sh_item + 1] > s_cum[sh_item]) {
        int first, last;
        item_units(geo, shape.switch_quanta, s_cum[sh_item], s_cum[sh_item + 1], first, last);
        r[2] = first;
        r[3] = last - first + 1;
      }
    }
    *reinterpret_cast<int4_t*>(pp.rows + 4 * static_cast<int64_t>(b)) = r;
  }
  for (int u = tid; u < pp.num_units; u += kPlanThreads) {
    int rec[kPlanUnitWords];
#pragma unroll
    for (int i = 0; i < kPlanUnitWords; ++i) rec[i] = 0;
    const int q0 = geo.unit_start(u), q1 = geo.unit_start(u + 1);
    TileCursor c;
    if (q0 < q1 && cursor_seek(c, table, shape.switch_quanta, num_items, q0, q1)) {
      rec[kPuQ0] = q0;
      rec[kPuQ1] = q1;
      rec[kPuItem] = c.b;
      rec[kPuTok] = c.tok;
      rec[kPuSegEnd] = c.seg_end;
      rec[kPuQEnd] = c.q_end;
      rec[kPuLo] = c.it.lo;
      rec[kPuEnd] = c.it.end;
      rec[kPuRow] = c.it.row;
      rec[kPuNseq] = c.it.nseq;
      // block ids of the first tile's columns; columns behind the segment's last one repeat it
      const int col0 = c.tok / pp.block_size;
      int last = (c.seg_end - 1) / pp.block_size;
      last = last < pp.max_blocks - 1 ? last : pp.max_blocks - 1;
      const int32_t* table_row = pp.block_table + static_cast<int64_t>(c.it.row) * pp.max_blocks;
#pragma unroll
      for (int i = 0; i < kPlanUnitIds; ++i) rec[kPuIds + i] = table_row[col0 + i < last ? col0 + i : last];
    }
    int4_t* dst = reinterpret_cast<int4_t*>(pp.units + static_cast<int64_t>(u) * kPlanUnitWords);
#pragma unroll
    for (int i = 0; i < kPlanUnitWords / 4; ++i) dst[i] = int4_t{rec[4 * i], rec[4 * i + 1], rec[4 * i + 2], rec[4 * i + 3]};
  }
}

// layout of a plan buffer for an item list of `items` entries and `units` units, in int32 words
struct PlanLayout {
  size_t cum, items, units, rows, words;
};
PlanLayout plan_layout(size_t items, size_t units, size_t batch) {
  PlanLayout l;
  l.cum = 0;
  l.items = (items + 1 + 3) / 4 * 4;  // 16-byte aligned
  l.units = l.items + 4 * items;
  l.rows = l.units + kPlanUnitWords * units + 4;  // (the four words in front of the rows: total cost positions, 0, 0, 0)
  l.words = l.rows + 4 * batch;
  return l;
}

int decode_impl(const areno_paged_cache* cache, const void* q, const void* k_update, const void* v_update, void* out,
                int32_t q_dtype, int32_t batch, int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits, float softmax_scale,
                int32_t group_rows, const int32_t* shared_lens, const areno_decode_plan* plan, void* workspace,
                size_t workspace_bytes, int32_t stages, void* stream) {
  const char* op = "areno_hip_paged_decode";
  if (int rc = validate_paged_cache(cache, op)) return rc;
  if (q == nullptr || out == nullptr || block_table == nullptr || cache_seqlens == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: q/out/block_table/cache_seqlens is NULL", op);
  if ((k_update == nullptr) != (v_update == nullptr))
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: k_update and v_update must both be given or both be NULL", op);
  if (batch < 0 || batch > 65535 || q_heads <= 0 || max_blocks <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: batch/q_heads/max_blocks out of range", op);
  if (q_heads % cache->kv_heads != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: q heads must be divisible by kv heads", op);
  if (num_splits < 1) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: num_splits must be >= 1", op);
  if (q_dtype != ARENO_DT_F32 && q_dtype != ARENO_DT_F16 && q_dtype != ARENO_DT_BF16)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: q must be f32, f16 or bf16", op);
  if (!is_quantized(cache->cache_dtype) && cache->cache_dtype != q_dtype)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: q dtype must equal an unquantized cache's dtype", op);
  if (cache->head_dim > kGenericMaxPerLane * kWave)
    return fail(ARENO_ERR_UNSUPPORTED, "%s: head_dim %d > %d", op, cache->head_dim, kGenericMaxPerLane * kWave);
  if (batch == 0) return ARENO_OK;

  Chunking ch;
  if (!pick_chunking(cache->block_size, max_blocks, num_splits, &ch))
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: block_size * max_blocks out of range", op);
  const size_t base_need = areno_hip_paged_decode_workspace_bytes(batch, q_heads, cache->head_dim, cache->block_size,
                                                                  max_blocks, num_splits);
  MfmaChoice choice = choose_mfma(cache, q_dtype, batch, q_heads, window_left, k_update != nullptr, group_rows,
                                  shared_lens != nullptr);
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) choice.fn = nullptr;
  const int num_shared = choice.fn != nullptr ? choice.items.num_shared : 0;
  const size_t plan_extra = num_shared > 0 ? grouped_plan_bytes(batch) : 0;
  const size_t need =
      base_need + plan_extra + (num_shared > 0 ? shared_region_bytes(cache->kv_heads, cache->head_dim, num_shared) : 0);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(ARENO_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", op, need, workspace_bytes);

  // a plan must have been built for exactly this call's shapes (its tables are read without further checks)
  const bool planned = plan != nullptr && plan->units > 0;
  if (planned) {
    const int32_t eff_group_rows = num_shared > 0 ? group_rows : 0;
    if (choice.fn == nullptr || plan->buffer == nullptr || plan->batch != batch || plan->q_heads != q_heads ||
        plan->kv_heads != cache->kv_heads || plan->head_dim != cache->head_dim || plan->block_size != cache->block_size ||
        plan->max_blocks != max_blocks || plan->window_left != window_left || plan->cache_dtype != cache->cache_dtype ||
        plan->q_dtype != q_dtype || plan->with_update != (k_update != nullptr ? 1 : 0) ||
        plan->group_rows != eff_group_rows || plan->units != choice.grid.units ||
        plan->items != choice.items.num_items() || plan->tile_tokens != choice.tile_tokens)
      return fail(ARENO_ERR_INVALID_ARGUMENT,
                  "%s: the plan was built for other shapes (batch, heads, head_dim, page size, table width, window, "
                  "cache / query dtype, update rows or prefix groups differ)", op);
  }

  DecodeParams p;
  p.q = q;
  p.k_cache = cache->k;
  p.v_cache = cache->v;
  p.k_scale = cache->k_scale;
  p.v_scale = cache->v_scale;
  p.block_table = block_table;
  p.cache_seqlens = cache_seqlens;
  const size_t rows = static_cast<size_t>(batch) * q_heads * ch.max_parts;
  p.part_ml = static_cast<float*>(workspace);
  p.part_acc = p.part_ml + rows * 2;
  p.out = out;
  p.batch = batch;
  p.q_heads = q_heads;
  p.kv_heads = cache->kv_heads;
  p.head_dim = cache->head_dim;
  p.block_size = cache->block_size;
  p.bs_shift = log2_exact(cache->block_size);
  p.max_blocks = max_blocks;
  p.window_left = window_left;
  p.chunk = ch.chunk;
  p.max_parts = ch.max_parts;
  p.q_dtype = q_dtype;
  p.cache_dtype = cache->cache_dtype;
  p.scale_dtype = cache->scale_dtype;
  p.group = q_heads / cache->kv_heads;
  p.heads_per_wg = cache->kv_heads % 4 == 0 ? 4 : (cache->kv_heads % 2 == 0 ? 2 : 1);
  p.scale_log2e = softmax_scale * kLog2e;

  hipStream_t s = static_cast<hipStream_t>(stream);
  const decode_mfma_fn mfma = choice.fn;
  const MfmaGrid& grid = choice.grid;
  // ---- append: the merge launch of the matrix-core path does it (append_in_merge); a launch of its own in front of
  // the other kernels, and for a staged call that asks for the append without the merge ------------------------------
  const bool merge_appends = mfma != nullptr && choice.items.append_in_merge != 0;
  const bool append_in_front = k_update != nullptr && (stages & ARENO_STAGE_APPEND) &&
                               (!merge_appends || !(stages & ARENO_STAGE_REDUCE));
  if (append_in_front) {
    if (int rc = areno_hip_cache_write_decode(cache, k_update, v_update, q_dtype, batch, block_table, max_blocks,
                                              cache_seqlens, stream))
      return rc;
  }

  if (mfma != nullptr) {
    MfmaDecodeParams mp;
    mp.d = p;
    mp.d.heads_per_wg = grid.heads_per_wg;
    mp.tok_splits = grid.tok_splits;
    mp.num_units = grid.units;
    mp.head_parts = choice.head_parts;
    {
      PageDivision division = {0, 0};
      page_division(cache->block_size, &division);  // (checked by choose_mfma)
      mp.bs_magic = division.magic;
      mp.bs_post = division.post;
    }
    mp.items = choice.items;
    mp.k_update = merge_appends ? k_update : nullptr;
    mp.v_update = merge_appends ? v_update : nullptr;
    mp.write_append = (merge_appends && (stages & ARENO_STAGE_APPEND) && !append_in_front) ? 1 : 0;
    mp.num_blocks = cache->num_blocks;
    mp.trace = g_trace_buffer;
    const size_t slots = static_cast<size_t>(grid.units) + batch;
    const size_t part_bytes = mfma_partial_bytes(slots, q_heads, p.head_dim);
    mp.d.part_ml = static_cast<float*>(workspace);
    mp.d.part_acc = mp.d.part_ml + slots * q_heads * 2;
    mp.dump = mp.d.part_acc + slots * q_heads * p.head_dim;
    mp.cum_out = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + part_bytes);
    mp.shared_lens = shared_lens;
    mp.shared_ml = nullptr;
    mp.shared_acc = nullptr;
    if (num_shared > 0) {
      // behind the ungrouped layout: the (longer) prefix sums of the item list, then the shared partial region
      mp.cum_out = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + base_need);
      char* region = static_cast<char*>(workspace) + base_need + plan_extra;
      const size_t shared_slots = static_cast<size_t>(grid.units) + num_shared;
      mp.shared_ml = reinterpret_cast<float*>(region);
      mp.shared_acc = mp.shared_ml + shared_slots * cache->kv_heads * 16 * 2;
    }
    mp.plan_cum = nullptr;
    mp.plan_items = nullptr;
    mp.plan_units = nullptr;
    mp.plan_rows = nullptr;
    if (planned) {
      const PlanLayout l = plan_layout(plan->items, plan->units, plan->batch);
      const int32_t* words = static_cast<const int32_t*>(plan->buffer);
      mp.plan_cum = words + l.cum;
      mp.plan_items = words + l.items;
      mp.plan_units = words + l.units;
      mp.plan_rows = words + l.rows;
    }
    if (stages & ARENO_STAGE_SPLIT) {
      hipLaunchKernelGGL(mfma, dim3(grid.workgroups, grid.head_groups), dim3(grid.waves * kWave), 0, s, mp.plan_units,
                         mp.plan_items, mp.plan_cum, p.cache_seqlens, mp.tok_splits, mp.d.heads_per_wg,
                         mp.items.num_items(), mp);
      if (int rc = check_launch(op)) return rc;
    }
    if (stages & ARENO_STAGE_REDUCE) {
      // (q_dtype is F16 or BF16 on this path; h / group as a multiplication: exact for h < 2^16)
      const uint32_t group_magic = p.group > 1 ? static_cast<uint32_t>((uint64_t{1} << 32) / p.group + 1) : 0u;
      const int merge_waves = merge_waves_for(grid.units, batch);
      const reduce_slots_fn merge =
          reduce_slots_kernel_for(p.head_dim, q_dtype, cache->cache_dtype, mp.plan_rows != nullptr, merge_waves);
      const dim3 merge_grid(merge_waves == 1 ? (q_heads + kReduceRows - 1) / kReduceRows : q_heads, batch);
      hipLaunchKernelGGL(merge, merge_grid, dim3((merge_waves == 1 ? kReduceRows : merge_waves) * kWave), 0, s,
                         mp.plan_rows, p.cache_seqlens, p.q, mp.k_update, mp.v_update, q_heads, p.kv_heads, p.group,
                         group_magic, p.head_dim, mp);
      if (int rc = check_launch(op)) return rc;
    }
    return ARENO_OK;
  }

  decode_split_fn fast = nullptr;
  const bool aligned = (reinterpret_cast<uintptr_t>(cache->k) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(cache->v) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(workspace) % 16 == 0);
  if (aligned && q_dtype != ARENO_DT_F32) {
    switch (cache->cache_dtype) {
      case ARENO_DT_BF16: fast = decode_split_lookup_bf16(p.head_dim, p.group); break;
      case ARENO_DT_F16: fast = decode_split_lookup_f16(p.head_dim, p.group); break;
      case ARENO_DT_I8: fast = decode_split_lookup_i8(p.head_dim, p.group); break;
      case ARENO_DT_FP8_E4M3: fast = decode_split_lookup_fp8(p.head_dim, p.group); break;
      default: break;
    }
  }
  if (!(stages & ARENO_STAGE_SPLIT)) {
    // skip
  } else if (fast != nullptr) {
    const dim3 grid3(ch.max_parts, batch, cache->kv_heads / p.heads_per_wg);
    hipLaunchKernelGGL(fast, grid3, dim3(kDecodeThreads), 0, s, p);
  } else {
    const dim3 grid3(batch * q_heads, ch.max_parts);
    hipLaunchKernelGGL(decode_split_generic_kernel, grid3, dim3(kWave), 0, s, p);
  }
  if (int rc = check_launch(op)) return rc;
  if (!(stages & ARENO_STAGE_REDUCE)) return ARENO_OK;
  const int rblocks = (batch * q_heads + kReduceRows - 1) / kReduceRows;
  hipLaunchKernelGGL(decode_reduce_kernel, dim3(rblocks), dim3(kReduceRows * kWave), 0, s, p);
  return check_launch(op);
}

}  // namespace
}  // namespace areno

namespace areno {
namespace {

// Batches beyond what one launch of the matrix-core kernel indexes (kMfmaMaxBatch rows: its prefix sum over the rows
// lives in LDS) run as consecutive launches over row ranges, on the same stream and through the same workspace.
int decode_in_row_ranges(const areno_paged_cache* cache, const void* q, const void* k_update, const void* v_update,
                         void* out, int32_t q_dtype, int32_t batch, int32_t q_heads, const int32_t* block_table,
                         int32_t max_blocks, const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                         float softmax_scale, int32_t group_rows, const int32_t* shared_lens,
                         const areno_decode_plan* plan, void* workspace, size_t workspace_bytes, int32_t stages,
                         void* stream) {
  if (batch <= kMfmaMaxBatch || cache == nullptr || q == nullptr || out == nullptr || block_table == nullptr ||
      cache_seqlens == nullptr || q_heads <= 0 || max_blocks <= 0 || cache->kv_heads <= 0 || cache->head_dim <= 0)
    return decode_impl(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table, max_blocks,
                       cache_seqlens, window_left, num_splits, softmax_scale, group_rows, shared_lens, plan, workspace,
                       workspace_bytes, stages, stream);
  // (a plan covers one launch: areno_hip_paged_decode_plan leaves units = 0 for batches this large)
  int rows_per_launch = kMfmaMaxBatch;
  if (shared_lens != nullptr && group_rows > 1) rows_per_launch = kMfmaMaxBatch / group_rows * group_rows;
  if (rows_per_launch <= 0) rows_per_launch = kMfmaMaxBatch;  // groups wider than a launch: decode_impl drops the hint
  const size_t es = dtype_size(q_dtype);
  const size_t q_row = static_cast<size_t>(q_heads) * cache->head_dim * es;
  const size_t kv_row = static_cast<size_t>(cache->kv_heads) * cache->head_dim * es;
  for (int32_t r0 = 0; r0 < batch; r0 += rows_per_launch) {
    const int32_t rows = batch - r0 < rows_per_launch ? batch - r0 : rows_per_launch;
    const bool grouped = shared_lens != nullptr && group_rows > 1 && rows_per_launch % group_rows == 0;
    const int rc = decode_impl(
        cache, static_cast<const char*>(q) + r0 * q_row,
        k_update != nullptr ? static_cast<const char*>(k_update) + r0 * kv_row : nullptr,
        v_update != nullptr ? static_cast<const char*>(v_update) + r0 * kv_row : nullptr,
        static_cast<char*>(out) + r0 * q_row, q_dtype, rows, q_heads, block_table + static_cast<size_t>(r0) * max_blocks,
        max_blocks, cache_seqlens + r0, window_left, num_splits, softmax_scale, grouped ? group_rows : 1,
        grouped ? shared_lens + r0 / group_rows : nullptr, nullptr, workspace, workspace_bytes, stages, stream);
    if (rc != ARENO_OK) return rc;
  }
  return ARENO_OK;
}

}  // namespace
}  // namespace areno

extern "C" int areno_hip_paged_decode_stages(const areno_paged_cache* cache, const void* q, const void* k_update,
                                             const void* v_update, void* out, int32_t q_dtype, int32_t batch,
                                             int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                             const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                                             float softmax_scale, void* workspace, size_t workspace_bytes,
                                             int32_t stages, void* stream) {
  return areno::decode_in_row_ranges(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table, max_blocks,
                            cache_seqlens, window_left, num_splits, softmax_scale, 0, nullptr, nullptr, workspace,
                            workspace_bytes, stages, stream);
}

extern "C" size_t areno_hip_paged_decode_grouped_workspace_bytes(int32_t batch, int32_t q_heads, int32_t kv_heads,
                                                                 int32_t head_dim, int32_t block_size,
                                                                 int32_t max_blocks, int32_t num_splits,
                                                                 int32_t group_rows) {
  const size_t base = areno_hip_paged_decode_workspace_bytes(batch, q_heads, head_dim, block_size, max_blocks, num_splits);
  if (base == 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return 0;
  int cols_seqs = 0, subs_per_group = 0;
  const int num_shared = areno::shared_items_for(batch, q_heads / kv_heads, group_rows, &cols_seqs, &subs_per_group);
  if (num_shared == 0) return base;
  return base + areno::grouped_plan_bytes(batch) + areno::shared_region_bytes(kv_heads, head_dim, num_shared);
}

extern "C" int areno_hip_paged_decode_grouped(const areno_paged_cache* cache, const void* q, const void* k_update,
                                              const void* v_update, void* out, int32_t q_dtype, int32_t batch,
                                              int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                              const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                                              float softmax_scale, int32_t group_rows, const int32_t* shared_lens,
                                              void* workspace, size_t workspace_bytes, int32_t stages, void* stream) {
  if (shared_lens != nullptr && (group_rows < 1 || (batch > 0 && batch % group_rows != 0)))
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT,
                       "areno_hip_paged_decode_grouped: batch %d is not a multiple of group_rows %d", batch, group_rows);
  return areno::decode_in_row_ranges(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table, max_blocks,
                            cache_seqlens, window_left, num_splits, softmax_scale, group_rows, shared_lens, nullptr,
                            workspace, workspace_bytes, stages, stream);
}

extern "C" size_t areno_hip_paged_decode_plan_bytes(int32_t batch) {
  if (batch <= 0) return 0;
  const size_t items = 2 * static_cast<size_t>(batch < areno::kMfmaMaxBatch ? batch : areno::kMfmaMaxBatch);
  return areno::plan_layout(items, areno::kMfmaMaxUnits, items / 2).words * sizeof(int32_t);
}

extern "C" int areno_hip_paged_decode_plan(areno_decode_plan* plan, void* buffer, size_t buffer_bytes,
                                           const areno_paged_cache* cache, int32_t q_dtype, int32_t batch,
                                           int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                           const int32_t* cache_seqlens, int32_t window_left, int32_t with_update,
                                           int32_t group_rows, const int32_t* shared_lens, void* stream) {
  using namespace areno;
  const char* op = "areno_hip_paged_decode_plan";
  if (plan == nullptr) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: plan is NULL", op);
  if (int rc = validate_paged_cache(cache, op)) return rc;
  if (block_table == nullptr || cache_seqlens == nullptr || batch < 0 || q_heads <= 0 || max_blocks <= 0 ||
      q_heads % cache->kv_heads != 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL block_table / cache_seqlens or sizes out of range", op);
  if (shared_lens != nullptr && (group_rows < 1 || (batch > 0 && batch % group_rows != 0)))
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: batch %d is not a multiple of group_rows %d", op, batch, group_rows);
  const MfmaChoice choice = batch > 0 ? choose_mfma(cache, q_dtype, batch, q_heads, window_left, with_update != 0,
                                                    group_rows, shared_lens != nullptr)
                                      : MfmaChoice{};
  plan->buffer = buffer;
  plan->buffer_bytes = buffer_bytes;
  plan->batch = batch;
  plan->q_heads = q_heads;
  plan->kv_heads = cache->kv_heads;
  plan->head_dim = cache->head_dim;
  plan->block_size = cache->block_size;
  plan->max_blocks = max_blocks;
  plan->window_left = window_left;
  plan->cache_dtype = cache->cache_dtype;
  plan->q_dtype = q_dtype;
  plan->with_update = with_update != 0 ? 1 : 0;
  plan->group_rows = 0;
  plan->units = 0;
  plan->items = 0;
  plan->tile_tokens = 0;
  if (batch == 0 || choice.fn == nullptr) return ARENO_OK;  // a kernel that takes no plan serves these shapes
  const PlanLayout l = plan_layout(choice.items.num_items(), choice.grid.units, batch);
  if (buffer == nullptr || reinterpret_cast<uintptr_t>(buffer) % 16 != 0 || buffer_bytes < l.words * sizeof(int32_t))
    return fail(ARENO_ERR_WORKSPACE, "%s: a 16-byte aligned buffer of %zu bytes is needed, %zu given", op,
                l.words * sizeof(int32_t), buffer_bytes);
  PlanParams pp;
  pp.cache_seqlens = cache_seqlens;
  pp.shared_lens = shared_lens;
  pp.block_table = block_table;
  int32_t* words = static_cast<int32_t*>(buffer);
  pp.cum = words + l.cum;
  pp.items = words + l.items;
  pp.units = words + l.units;
  pp.rows = words + l.rows;
  pp.shape = choice.items;
  pp.num_units = choice.grid.units;
  pp.block_size = cache->block_size;
  pp.max_blocks = max_blocks;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (choice.items.num_shared > 0) {
    hipLaunchKernelGGL(decode_plan_kernel<true>, dim3(1), dim3(kPlanThreads), 0, s, pp);
  } else {
    hipLaunchKernelGGL(decode_plan_kernel<false>, dim3(1), dim3(kPlanThreads), 0, s, pp);
  }
  if (int rc = check_launch(op)) return rc;
  plan->group_rows = choice.items.num_shared > 0 ? group_rows : 0;
  plan->units = choice.grid.units;
  plan->items = choice.items.num_items();
  plan->tile_tokens = choice.tile_tokens;
  return ARENO_OK;
}

extern "C" int areno_hip_paged_decode_planned(const areno_paged_cache* cache, const void* q, const void* k_update,
                                              const void* v_update, void* out, int32_t q_dtype, int32_t batch,
                                              int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                              const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                                              float softmax_scale, int32_t group_rows, const int32_t* shared_lens,
                                              const areno_decode_plan* plan, void* workspace, size_t workspace_bytes,
                                              int32_t stages, void* stream) {
  if (shared_lens != nullptr && (group_rows < 1 || (batch > 0 && batch % group_rows != 0)))
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT,
                       "areno_hip_paged_decode_planned: batch %d is not a multiple of group_rows %d", batch, group_rows);
  return areno::decode_in_row_ranges(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table, max_blocks,
                            cache_seqlens, window_left, num_splits, softmax_scale, group_rows, shared_lens, plan,
                            workspace, workspace_bytes, stages, stream);
}

// ---- the decode op for callers that cannot allocate -----------------------------------------------------------------
// The split-KV partials of areno_hip_paged_decode_static live in this array instead of a caller workspace.  Every
// GPU the library runs on holds its own copy, at its own address, until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress: the device address is looked up once per device and kept, and that
// pointer is what the kernels receive.
#define ARENO_STATIC_SCRATCH_BYTES (64u << 20)
static __device__ __align__(256) unsigned char scratch[ARENO_STATIC_SCRATCH_BYTES];

namespace areno {
namespace {

constexpr int kMaxScratchDevices = 64;

// Device address of `scratch` on the current device (looked up at the first call on that device), or NULL with the
// error recorded.
void* static_scratch(const char* op) {
  static std::mutex lock;
  static void* address[kMaxScratchDevices] = {};
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess || device < 0 || device >= kMaxScratchDevices) {
    fail(ARENO_ERR_LAUNCH, "%s: no current device (%s)", op, hipGetErrorString(err));
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(lock);
  if (address[device] == nullptr) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      fail(ARENO_ERR_LAUNCH, "%s: the built-in scratch buffer has no address on device %d (%s)", op, device,
           hipGetErrorString(err));
      return nullptr;
    }
    address[device] = ptr;
  }
  return address[device];
}

}  // namespace
}  // namespace areno

extern "C" size_t areno_hip_paged_decode_static_capacity(void) { return ARENO_STATIC_SCRATCH_BYTES; }

extern "C" int areno_hip_paged_decode_static(const areno_paged_cache* cache, const void* q, const void* k_update,
                                             const void* v_update, void* out, int32_t q_dtype, int32_t batch,
                                             int32_t q_heads, const int32_t* block_table, int32_t max_blocks,
                                             const int32_t* cache_seqlens, int32_t window_left, int32_t num_splits,
                                             float softmax_scale, void* stream) {
  const char* op = "areno_hip_paged_decode_static";
  if (cache == nullptr) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: cache is NULL", op);
  if (batch == 0) return ARENO_OK;
  const size_t need = areno_hip_paged_decode_workspace_bytes(batch, q_heads, cache->head_dim, cache->block_size,
                                                             max_blocks, num_splits);
  if (need == 0) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: batch/q_heads/head_dim/max_blocks out of range", op);
  if (need > ARENO_STATIC_SCRATCH_BYTES)
    return areno::fail(ARENO_ERR_WORKSPACE,
                       "%s: these shapes need %zu bytes for the split-KV partials, the built-in buffer holds %zu; call "
                       "areno_hip_paged_decode with a workspace of the caller's",
                       op, need, static_cast<size_t>(ARENO_STATIC_SCRATCH_BYTES));
  void* ptr = areno::static_scratch(op);
  if (ptr == nullptr) return ARENO_ERR_LAUNCH;
  // every partial, prefix sum and plan entry a launch reads was written earlier in the same launch sequence, so
  // nothing left by the previous call has to be cleared
  return areno_hip_paged_decode_stages(cache, q, k_update, v_update, out, q_dtype, batch, q_heads, block_table,
                                       max_blocks, cache_seqlens, window_left, num_splits, softmax_scale, ptr,
                                       ARENO_STATIC_SCRATCH_BYTES, ARENO_STAGE_ALL, stream);
}

#ifdef ARENO_TRACE
// Tuning builds only: a device buffer of [waves][8] 64-bit words that the split kernel fills with its wave timestamps.
extern "C" void areno_hip_debug_set_trace(void* device_buffer) {
  areno::g_trace_buffer = static_cast<unsigned long long*>(device_buffer);
}
#endif
