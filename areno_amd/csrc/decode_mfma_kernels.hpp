// Split-KV GQA paged decode on the matrix cores (gfx950), device code.
//
// Why MFMA for a bandwidth-bound op: at 70 % of 8 TB/s every SIMD must consume ~2.3 KV bytes per clock
// and each int8/fp8 byte needs G = q_heads / kv_heads multiply-adds on the QK^T side and G more on the P.V
// side.  With G = 7 that is more than the vector ALU can issue even with v_dot2, so the VALU kernel
// (paged_decode_kernels.hpp) tops out well below the HBM roofline.  Here the G query heads of one KV head
// form the (zero padded) 16-wide N side of v_mfma_f32_16x16x32 tiles; the vector ALU only dequantizes
// (<= 0.75 op per element) and runs the softmax.
//
// Work decomposition (exactly balanced, no host knowledge of the lengths):
//   * a sequence contributes ceil(visible_keys / 32) tiles of 32 tokens; every workgroup computes the
//     prefix sum of tile counts over the batch in LDS and takes an equal share of the global tile range
//     ("wave piece"), so all waves stream the same number of bytes whatever the length distribution;
//   * a piece that crosses a sequence boundary emits one partial per sequence it touches, into slot
//     (piece index + sequence index), which is unique and contiguous per sequence; the reduce kernel merges
//     the slots of each sequence.
//   * block = 4 wave64; wave w owns KV head z*HW + w % HW, so with kv_heads >= 4 the four waves of a
//     workgroup read whole pages ([slot][kv_head][D] is contiguous).  Waves never synchronise after the
//     prefix sum: each has private LDS tiles.
// Data path per 32-token tile and wave:
//   global --16 B/lane coalesced loads--> registers (in flight while the previous tile is computed)
//          --ds_write_b128--> LDS K tile [32][D*es + 16] and V tile (row padding makes every access below
//          bank-conflict free)
//   S^T[token][head] = K . Q^T : A = K rows read straight from LDS (8 consecutive dims per lane), B = Q^T held in
//          registers for the whole sequence; C puts head = lane % 16, 4 tokens per lane.
//   online softmax in the log2 domain on C; the per-token K scale multiplies S, the V scale multiplies P.
//   O^T[dim][head] += V^T . P^T : A = V^T through ds_read_b64_tr_b8 / _tr_b16 (the LDS transpose read gives each
//          lane 8 tokens of one dim), B = P^T which *is* the C layout of S^T (token order chosen to match), so
//          no cross-lane movement of P is needed.
// int8 codes become fp16 by placing (code ^ 0x80) under the exponent byte 0x64 (v_perm): 1152 + code exactly;
// the offsets are removed algebraically (1152 * sum(q) per head, 1152 * sum(p) per head).  fp8 uses
// v_cvt_scalef32_pk_f16_fp8 with scale 1 (exact).  bf16 / fp16 caches feed the MFMA directly.
//
// The single-token append (areno/accel/csrc/attention.cu:526-553) rides along: the wave that stages the last tile of a
// sequence takes the newest token's row from k_update / v_update instead of the not yet written page slot, quantizes
// it with the cache writer's closed form and stores it into the page.
//
// GROUPED instantiation (batches whose rows come in prefix groups, e.g. the samples of one prompt): the item list is
// [shared prefix of every sub-group of rows that fits side by side in the 16 MFMA columns] + [the rest of every
// row]; a shared item is streamed once with column = (row in sub-group, head) and leaves its partials in a second
// region, the merge kernel adds them to the row's own.
//
// Semantics: the reference's split kernel (areno/accel/csrc/attention.cu:555-654) -- keys [first_allowed, L_b],
// q head h <-> kv head h / G, fp32 accumulation.
#pragma once

#include <type_traits>

#include "paged_decode_kernels.hpp"

namespace areno {

constexpr int kMfmaMaxBatch = 1024;  // prefix-sum capacity of one workgroup
#ifndef ARENO_MFMA_NW
#define ARENO_MFMA_NW 4
#endif
constexpr int kTileTokens = 32;

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) int int2_t;

struct MfmaDecodeParams {
  DecodeParams d;      // part_ml / part_acc are indexed [slot][q_head] here
  int32_t* plan;         // [batch + 1]: exclusive prefix sums of tiles per sequence (written by workgroup 0)
  int32_t tok_splits;    // waves of a workgroup that share a KV head (waves per workgroup / heads_per_wg)
  int32_t static_wgs;    // workgroups [0, static_wgs) own the big units, the rest of the grid the small ones
  int32_t num_pieces;    // static_wgs * tok_splits: big units
  int32_t max_small;     // (gridDim.x - static_wgs) * tok_splits: small units available
  int32_t static_share;  // n/256 of all tiles go to the big units
  int32_t min_unit_tiles;
  // Fused append: when set, the wave that stages the last tile of a sequence takes the newest token's K / V row
  // from here ([batch, kv_heads, head_dim], dtype q_dtype) instead of the cache, quantizes it like the cache
  // writer and stores it (and its scales) into the page, so no separate append launch is needed.
  const void* k_update;
  const void* v_update;
  // Prefix groups (GROUPED kernels only): rows [i * group_rows, (i + 1) * group_rows) share the pages of their first
  // shared_lens[i] tokens (an RL rollout's samples of one prompt).  Those tokens become "shared items" that are read
  // once for up to cols_seqs = 16 / q-heads-per-kv-head sequences side by side in the 16 MFMA columns; the rest of
  // each sequence is an item of its own.  Shared items leave their partials in a second region (16 columns per kv
  // head and slot).
  const int32_t* shared_lens;  // [batch / group_rows]
  int32_t group_rows;          // rows per prefix group
  int32_t cols_seqs;           // sequences that fit side by side: 16 / group
  int32_t subs_per_group;      // ceil(group_rows / cols_seqs)
  int32_t num_shared;          // shared items: (batch / group_rows) * subs_per_group, listed before the per-row items
  float* shared_ml;            // [slot][kv_head][16][2]
  float* shared_acc;           // [slot][kv_head][16][head_dim]
#ifdef ARENO_TRACE
  unsigned long long* trace;  // [wave][16] timestamps, tuning builds only
#endif
};

template <int KIND>
struct MfmaOps;

template <>
struct MfmaOps<KV_BF16> {
  using vec8 = bf16x8_t;
  static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct MfmaOps<KV_F16> {
  using vec8 = half8_t;
  static __device__ __forceinline__ float4_t mfma(vec8 a, vec8 b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct MfmaOps<KV_I8> : MfmaOps<KV_F16> {};
template <>
struct MfmaOps<KV_FP8> : MfmaOps<KV_F16> {};

typedef __attribute__((address_space(3))) int2_t lds_int2;
typedef __attribute__((address_space(3))) short4_t lds_short4;

// 8 elements (two dwords of 8-bit codes, or four dwords of 16-bit values) -> one MFMA operand register group
template <int KIND>
__device__ __forceinline__ typename MfmaOps<KIND>::vec8 to_operand(const uint32_t* w) {
  using V = typename MfmaOps<KIND>::vec8;
  uint4_t r;
  if constexpr (KIND == KV_BF16 || KIND == KV_F16) {
    r = uint4_t{w[0], w[1], w[2], w[3]};
  } else if constexpr (KIND == KV_I8) {  // bytes already flipped to offset binary when staged
    r[0] = __builtin_amdgcn_perm(kF16Filler, w[0], 0x04010400u);
    r[1] = __builtin_amdgcn_perm(kF16Filler, w[0], 0x04030402u);
    r[2] = __builtin_amdgcn_perm(kF16Filler, w[1], 0x04010400u);
    r[3] = __builtin_amdgcn_perm(kF16Filler, w[1], 0x04030402u);
  } else {
    r[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[0], 1.0f, false));
    r[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[0], 1.0f, true));
    r[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[1], 1.0f, false));
    r[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[1], 1.0f, true));
  }
  return __builtin_bit_cast(V, r);
}

template <int KIND>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  using P = typename KVTraits<KIND>::pair_t;
  return __builtin_bit_cast(uint32_t, make_pair<P>(lo, hi));
}

// Quantize the 16 consecutive elements a lane holds of a new K or V row (32 raw bytes of 16-bit floats) exactly like
// the cache writer does (cache_write.hip): the row's abs-max is combined over the LPT lanes that share the row.
template <int KIND, bool SCALE16, int LPT>
__device__ __forceinline__ void quantize_row_chunk(const uint4_t (&raw)[2], int in_dtype, uint4_t& codes,
                                                   typename std::conditional<SCALE16, uint16_t, float>::type& scale_raw) {
  float x[16];
  float amax = 0.0f;
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    const uint32_t word = raw[w / 4][w % 4];
    if (in_dtype == ARENO_DT_BF16) {
      x[2 * w] = bf16_bits_to_float(word & 0xffffu);
      x[2 * w + 1] = bf16_bits_to_float(word >> 16);
    } else {
      x[2 * w] = f16_bits_to_float(word & 0xffffu);
      x[2 * w + 1] = f16_bits_to_float(word >> 16);
    }
    amax = fmaxf(amax, fmaxf(fabsf(x[2 * w]), fabsf(x[2 * w + 1])));
  }
#pragma unroll
  for (int m = 1; m < LPT; m <<= 1) amax = fmaxf(amax, wave_xor(amax, m));
  float s;
  if constexpr (KIND == KV_I8) {
    const _Float16 s16 = static_cast<_Float16>(fminf(amax / 127.0f, 65504.0f));
    const _Float16 s16_fixed = (s16 == static_cast<_Float16>(0.0f)) ? static_cast<_Float16>(1.0f) : s16;
    s = static_cast<float>(s16_fixed);
    if constexpr (SCALE16) {
      scale_raw = __builtin_bit_cast(uint16_t, s16_fixed);
    } else {
      scale_raw = s;
    }
  } else {
    s = amax / 448.0f;
    if (s == 0.0f) s = 1.0f;
    if constexpr (SCALE16) {
      scale_raw = static_cast<uint16_t>(float_to_f16_bits(s));
    } else {
      scale_raw = s;
    }
  }
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t byte;
      if constexpr (KIND == KV_I8) {
        const float code = fminf(fmaxf(rintf(x[4 * w + j] / s), -127.0f), 127.0f);
        byte = static_cast<uint32_t>(static_cast<int>(code)) & 0xffu;
      } else {
        byte = float_to_fp8_byte(fminf(fmaxf(x[4 * w + j] / s, -448.0f), 448.0f));
      }
      word |= byte << (8 * j);
    }
    codes[w] = word;
  }
}

// LDS row that holds tile token t of the V tile: the second half is rotated by 4 rows so that the 8 tokens a
// lane group reads through the transpose load ({4g..4g+3} and {16+4g..16+4g+3}) sit in rows distinct mod 16.
__device__ __forceinline__ int v_row_of(int t) { return t < 16 ? t : 16 + ((t + 4) & 15); }

// How the global tile range is cut into units (shared by the split and the reduce kernel).
struct UnitGeometry {
  int total_tiles;
  int static_tiles;  // tiles covered by the static units
  int static_units;  // one per wave piece
  int unit_tiles;    // tiles per small unit
  int small_units;
  // the products below fit 32 bits (every workload but the very largest): 32-bit divisions, which are a fifth of the
  // instructions of 64-bit ones and show in the launch-latency-sized reduce kernel
  bool narrow;

  __host__ __device__ int unit_start(int u) const {
    if (u <= static_units) {
      if (narrow)
        return static_cast<int>(static_cast<uint32_t>(u) * static_cast<uint32_t>(static_tiles) /
                                static_cast<uint32_t>(static_units));
      return static_cast<int>(static_cast<long long>(u) * static_tiles / static_units);
    }
    const long long x = static_tiles + static_cast<long long>(u - static_units) * unit_tiles;
    return x < total_tiles ? static_cast<int>(x) : total_tiles;
  }
  // unit that owns tile x (the largest unit whose first tile is <= x)
  __host__ __device__ int unit_of(int x) const {
    if (x < static_tiles) {
      if (narrow)
        return static_cast<int>((static_cast<uint32_t>(x + 1) * static_cast<uint32_t>(static_units) +
                                 static_cast<uint32_t>(static_tiles) - 1u) /
                                static_cast<uint32_t>(static_tiles)) -
               1;
      return static_cast<int>((static_cast<long long>(x + 1) * static_units + static_tiles - 1) / static_tiles - 1);
    }
    return static_units + (x - static_tiles) / unit_tiles;
  }
};

__host__ __device__ inline UnitGeometry make_unit_geometry(int total_tiles, int num_pieces, int max_small,
                                                           int static_share, int min_unit_tiles) {
  UnitGeometry g;
  g.total_tiles = total_tiles;
  g.static_units = num_pieces;
  g.static_tiles = static_cast<int>(static_cast<long long>(total_tiles) * static_share / 256);
  // short batches are not worth a tail of small units: everything goes to the big ones
  if (total_tiles < 4 * num_pieces || static_share >= 256 || max_small <= 0) g.static_tiles = total_tiles;
  const int rest = total_tiles - g.static_tiles;
  g.unit_tiles = min_unit_tiles < 1 ? 1 : min_unit_tiles;
  if (max_small > 0 && static_cast<long long>(g.unit_tiles) * max_small < rest)
    g.unit_tiles = (rest + max_small - 1) / max_small;
  g.small_units = (rest + g.unit_tiles - 1) / g.unit_tiles;
  // largest product in unit_start / unit_of: (static_tiles + 1) * static_units + static_tiles
  g.narrow = (static_cast<long long>(g.static_tiles) + 2) * (static_cast<long long>(num_pieces) + 1) < (1LL << 31);
  return g;
}

// Position of a tile stream inside a unit: which sequence, which token of it comes next.
// An item is a run of tokens [lo, hi) read through the block table of row `row`: a whole sequence's visible keys
// in the plain kernel; in a GROUPED kernel either the shared prefix of `nseq` adjacent rows or the rest of one row.
struct ItemInfo {
  int lo, hi, row, nseq;
};

struct TileCursor {
  int b;    // item (= sequence in the plain kernel)
  int tok;  // first token (position inside the sequence) of the tile
  int end;  // end of the item's token range (cache_seqlens[b] + 1 for a sequence)
  int row;  // block-table / query row of the item
  int nseq;
  ItemInfo next;  // item b + 1, fetched one item ahead
};

#ifndef ARENO_MFMA_QUANT_OCC
#define ARENO_MFMA_QUANT_OCC 2
#endif
// DSPLIT > 1 serves heads of DSPLIT * D elements (256 = 2 x 128, 192 = 3 x 64, 512 = 4 x 128): DSPLIT adjacent waves of the
// workgroup take one part of the head dimension each.  Every wave computes the part of S = K . Q^T over its
// elements, the waves exchange the parts through LDS (a wave's K tile is dead once its products are issued, so the
// part is parked there), add them in the same order and go on with identical scores: the same softmax in all,
// P . V over the wave's own part of V, the wave's part of the partial row.  The waves of a head synchronise through
// two counters each in LDS (part ready / parts consumed); no workgroup barrier is involved, so the heads of one
// workgroup may run different units.
template <int KIND, int D, bool SCALE16, int NW, bool GROUPED = false, int DSPLIT = 1>
__global__ __launch_bounds__(NW * kWave, KVTraits<KIND>::kQuant ? ARENO_MFMA_QUANT_OCC : 2) void decode_mfma_kernel(
    MfmaDecodeParams mp) {
  using T = KVTraits<KIND>;
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using Pair = typename T::pair_t;
  const DecodeParams& p = mp.d;
  constexpr int ES = T::kBytes;
  constexpr int EPL = 16 / ES;
  constexpr int LPT = D / EPL;
  constexpr int TPL = kWave / LPT;
  constexpr int TK = kTileTokens;
  constexpr int NLD = TK / TPL;  // 16-byte loads per lane, per tensor, per tile
  constexpr int RSK = D * ES + 16;
  constexpr int RSV = ES == 1 ? D + 16 : 2 * D + 32;
  constexpr int NS = D / 32;       // QK^T k-slices
  constexpr int NB = D / 16;       // P.V dim blocks
  constexpr int WPL = 8 * ES / 4;  // dwords per lane per k-slice of 8 elements
  constexpr float kPScale = T::kQuant ? 256.0f : 1.0f;
  constexpr int kWaveLds = TK * RSK + TK * RSV + 2 * TK * 4;
  static_assert(NLD >= 1 && LPT >= 4 && LPT <= 16, "unsupported head_dim");
  static_assert(DSPLIT == 1 || (DSPLIT >= 2 && DSPLIT <= 4 && !GROUPED && NW % DSPLIT == 0), "unsupported head split");
  constexpr int DFULL = D * DSPLIT;  // elements of a whole head (row of Q, of a cache page, of a partial)

  __shared__ __attribute__((aligned(16))) char s_tiles[NW][kWaveLds];
  constexpr int kMaxItems = (GROUPED ? 2 : 1) * kMfmaMaxBatch;  // at most one shared item per row on top of the rows
  __shared__ int s_cum[kMaxItems + 1];
  __shared__ int s_wave_tot[NW];
  // The length arrays in LDS: what a wave needs to know about an item comes from here instead of from a memory round
  // trip per lookup.  Without prefix groups the prefix sum's own loads fill s_len.  With them an item's extent takes up
  // to six dependent reads (the group's shared length, the members' lengths, the row's own) and the prefix sum asks for
  // 2 * 1024 / threads items per thread -- from global memory some forty round trips one after the other in the first
  // wave of every workgroup -- so the workgroup first copies both arrays with independent loads.  Where the copies
  // would cost the second resident workgroup (prefix groups over 16-bit caches) the lookups stay on global memory.
  constexpr bool kLocalLens = !GROUPED || ES == 1;
  constexpr int kMaxGroups = kMfmaMaxBatch / 2;  // groups have at least two rows
  __shared__ int s_len[kLocalLens ? kMfmaMaxBatch : 1];            // sequence lengths of the rows
  __shared__ int s_group_len[GROUPED && kLocalLens ? kMaxGroups : 1];  // shared prefix length of each group
  __shared__ int s_pair_flags[2][NW];  // [0]: score parts this wave has published, [1]: steps whose parts it has read
  constexpr int SPT = (kMaxItems + NW * kWave - 1) / (NW * kWave);  // items per thread in the prefix sum

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
#ifdef ARENO_TRACE
  const int trace_wave = (blockIdx.y * gridDim.x + blockIdx.x) * NW + wave;
  int trace_n = 2;
  if (mp.trace && lane == 0) {
    // start time, and in word 15 where the wave runs: XCC id (hardware register 20) above the HW_ID word (register 4)
    mp.trace[trace_wave * 16] = wall_clock64();
    mp.trace[trace_wave * 16 + 15] = (static_cast<unsigned long long>(__builtin_amdgcn_s_getreg((31 << 11) | 20)) << 32) |
                                     static_cast<unsigned int>(__builtin_amdgcn_s_getreg((31 << 11) | 4));
  }
#define ARENO_TRACE_POINT()                                                                   \
  if (mp.trace && lane == 0 && trace_n < 15) mp.trace[trace_wave * 16 + trace_n++] = wall_clock64()
#else
#define ARENO_TRACE_POINT()
#endif
  const int lr = lane & 15;  // MFMA row / column index
  const int lk = lane >> 4;  // MFMA k group
  const int grp = lane / LPT;
  const int dc = lane % LPT;

  // ---- the item list ----------------------------------------------------------------------------------------------
  const int num_items = GROUPED ? mp.num_shared + p.batch : p.batch;
  // tokens of a sub-group's shared prefix: the caller's figure, clipped to what every member has cached and cut to a
  // whole number of tiles
  if constexpr (GROUPED && kLocalLens) {
    // the launcher sends whole groups of at least two rows, at most kMfmaMaxBatch rows
    const int groups = min(p.batch / max(mp.group_rows, 2), kMaxGroups);
    for (int i = tid; i < min(p.batch, kMfmaMaxBatch); i += NW * kWave) s_len[i] = p.cache_seqlens[i];
    for (int i = tid; i < groups; i += NW * kWave) s_group_len[i] = mp.shared_lens[i];
    __syncthreads();
  }
  // length of row b / shared prefix length of group gi (indices clamped into the LDS copies)
  auto row_len = [&](int b) {
    if constexpr (GROUPED && kLocalLens) {
      return s_len[min(max(b, 0), kMfmaMaxBatch - 1)];
    } else {
      return p.cache_seqlens[b];
    }
  };
  auto group_len = [&](int gi) {
    if constexpr (GROUPED && kLocalLens) {
      return s_group_len[min(max(gi, 0), kMaxGroups - 1)];
    } else {
      return mp.shared_lens[gi];
    }
  };
  auto shared_tokens = [&](int sub, int& row0, int& count) {
    const int gi = sub / mp.subs_per_group;
    const int j = sub - gi * mp.subs_per_group;
    row0 = gi * mp.group_rows + j * mp.cols_seqs;
    count = min(mp.cols_seqs, mp.group_rows - j * mp.cols_seqs);
    int len = group_len(gi);
    for (int m = 0; m < count; ++m) len = min(len, row_len(row0 + m));
    return max(len, 0) & ~(TK - 1);
  };
  auto item_info = [&](int v) {
    ItemInfo it = {0, 0, 0, 1};
    if (v >= num_items) return it;
    if constexpr (GROUPED) {
      if (v < mp.num_shared) {
        it.hi = shared_tokens(v, it.row, it.nseq);
        return it;
      }
      const int b = v - mp.num_shared;
      const int gi = b / mp.group_rows;
      int row0, count;
      it.lo = shared_tokens(gi * mp.subs_per_group + (b - gi * mp.group_rows) / mp.cols_seqs, row0, count);
      it.hi = row_len(b) + 1;
      it.row = b;
      return it;
    } else {
      it.hi = s_len[v] + 1;
      it.lo = first_allowed_key(it.hi, p.window_left);
      it.row = v;
      return it;
    }
  };
  // ---- tiles per item, exclusive prefix sum over the items --------------------------------------------------------
  {
    int nt[SPT];
    int local = 0;
    if constexpr (GROUPED) {
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        nt[j] = 0;
        if (v < num_items) {
          const ItemInfo it = item_info(v);
          nt[j] = (it.hi - it.lo + TK - 1) / TK;
        }
        local += nt[j];
      }
    } else {
      // the thread's sequence lengths are fetched together (clamped index, no branch around the load): as loads
      // under `if (v < num_items)` they went out one at a time, SPT memory round trips at the start of every launch
      int len[SPT];
#pragma unroll
      for (int j = 0; j < SPT; ++j) len[j] = p.cache_seqlens[min(SPT * tid + j, num_items - 1)];
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        const int hi = len[j] + 1;
        nt[j] = v < num_items ? (hi - first_allowed_key(hi, p.window_left) + TK - 1) / TK : 0;
        if (v < num_items) s_len[v] = len[j];
        local += nt[j];
      }
    }
    int incl = local;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const int v = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += v;
    }
    if (lane == kWave - 1) s_wave_tot[wave] = incl;
    if (lane == 0) s_pair_flags[0][wave] = s_pair_flags[1][wave] = 0;
    __syncthreads();
    int excl = incl - local;
    for (int w2 = 0; w2 < wave; ++w2) excl += s_wave_tot[w2];
#pragma unroll
    for (int j = 0; j < SPT; ++j) {
      const int v = SPT * tid + j;
      if (v <= num_items) s_cum[v] = excl;
      excl += nt[j];
    }
    // the entry behind the last thread's items has no owner of its own: it is the total when the list is full
    if (tid == NW * kWave - 1 && SPT * (tid + 1) <= num_items) s_cum[SPT * (tid + 1)] = excl;
    __syncthreads();
  }
  // ---- unit geometry -----------------------------------------------------------------------------------
  // Tiles [0, static_tiles) are cut into num_pieces equal big units, one per wave of the first static_wgs
  // workgroups; the rest is cut into small units for the workgroups behind them in the grid.  Those start as CUs
  // become free, so the hardware dispatcher hands the tail to whichever CU got the better memory service:
  // service is uneven across CUs, and with equal shares only the slowest wave would set the run time.
  const int total_tiles = s_cum[num_items];
  const UnitGeometry geo =
      make_unit_geometry(total_tiles, mp.num_pieces, mp.max_small, mp.static_share, mp.min_unit_tiles);
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    for (int v = tid; v <= num_items; v += NW * kWave) mp.plan[v] = s_cum[v];
  }

  const int hw_count = p.heads_per_wg;
  const int half = wave % DSPLIT;  // which part of the head dimension this wave owns
  const int hw = (wave / DSPLIT) % hw_count;
  const int ts = (wave / DSPLIT) / hw_count;
  const int kvh = blockIdx.y * hw_count + hw;
  char* const k_tile = &s_tiles[wave][0];
  char* const v_tile = k_tile + TK * RSK;
  float* const ksc = reinterpret_cast<float*>(&s_tiles[wave][TK * RSK + TK * RSV]);
  float* const vsc = ksc + TK;

  constexpr int64_t row_bytes = static_cast<int64_t>(DFULL) * ES;
  const int64_t half_bytes = static_cast<int64_t>(half) * D * ES;  // of this wave's part inside a cache / update row
  const int h0 = kvh * p.group;
  const bool q_is_operand_type = (KIND == KV_BF16 && p.q_dtype == ARENO_DT_BF16) ||
                                 (KIND != KV_BF16 && p.q_dtype == ARENO_DT_F16);

  auto enter_item = [&](TileCursor& c, const ItemInfo& it) {
    c.tok = it.lo;
    c.end = it.hi;
    c.row = it.row;
    c.nseq = it.nseq;
  };
  // move a cursor from tile x to tile x + 1; returns true when that tile starts a new item
  auto advance = [&](TileCursor& c, int x_next) {
    if (x_next == s_cum[c.b + 1]) {
      ++c.b;
      if constexpr (GROUPED) {
        if (s_cum[c.b + 1] == x_next) {
          // items without tiles (a group with no shared prefix): skip them; the prefetched item is not the right one
          do {
            ++c.b;
          } while (s_cum[c.b + 1] == x_next);
          enter_item(c, item_info(c.b));
          c.next = item_info(c.b + 1);
          return true;
        }
      }
      enter_item(c, c.next);
      c.next = item_info(c.b + 1);
      return true;
    }
    c.tok += TK;
    return false;
  };
  auto is_shared = [&](int v) { return GROUPED && v < mp.num_shared; };

  TileCursor kv_cur, id_cur;
  int unit = 0;
  int ids[NLD];
  auto issue_id_loads = [&]() {
    const int32_t* table_row = p.block_table + static_cast<int64_t>(id_cur.row) * p.max_blocks;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int t = min(id_cur.tok + i * TPL + grp, id_cur.end - 1);
      const int col = p.bs_shift >= 0 ? (t >> p.bs_shift) : (t / p.block_size);
      ids[i] = table_row[col];
    }
  };

  uint4_t kreg[NLD], vreg[NLD];
  typedef typename std::conditional<SCALE16, uint16_t, float>::type scale_raw_t;
  scale_raw_t ksreg[NLD], vsreg[NLD];
  // fused append state of the tile in flight
  const bool fused_append = mp.k_update != nullptr;
  bool tail_tile = false;  // wave-uniform: the tile in kreg / vreg ends its sequence (holds the newest token)
  int64_t new_row = 0;     // cache row of the newest token, in the lanes that hold it
  uint4_t upd_k[2], upd_v[2];
  auto issue_kv_loads = [&]() {
    tail_tile = fused_append && !is_shared(kv_cur.b) && kv_cur.tok + TK >= kv_cur.end;
    const int64_t upd_row = static_cast<int64_t>(kv_cur.row) * p.kv_heads + kvh;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int tt = kv_cur.tok + i * TPL + grp;
      const int t = min(tt, kv_cur.end - 1);
      const int slot = p.bs_shift >= 0 ? (t & (p.block_size - 1)) : (t % p.block_size);
      const int64_t row = (static_cast<int64_t>(ids[i]) * p.block_size + slot) * p.kv_heads + kvh;
      const char* ka = static_cast<const char*>(p.k_cache) + row * row_bytes + half_bytes + dc * 16;
      const char* va = static_cast<const char*>(p.v_cache) + row * row_bytes + half_bytes + dc * 16;
      if (tail_tile && tt >= kv_cur.end - 1) {
        // the page slot of the newest token (and the clamped rows behind it) is not written yet
        if (tt == kv_cur.end - 1) new_row = row;
        if constexpr (!T::kQuant) {
          ka = static_cast<const char*>(mp.k_update) + upd_row * row_bytes + half_bytes + dc * 16;
          va = static_cast<const char*>(mp.v_update) + upd_row * row_bytes + half_bytes + dc * 16;
        }
      }
      kreg[i] = *reinterpret_cast<const uint4_t*>(ka);
      vreg[i] = *reinterpret_cast<const uint4_t*>(va);
      if constexpr (T::kQuant) {
        ksreg[i] = static_cast<const scale_raw_t*>(p.k_scale)[row];
        vsreg[i] = static_cast<const scale_raw_t*>(p.v_scale)[row];
      }
    }
    if constexpr (T::kQuant) {
      if (tail_tile) {
        // every lane group fetches the whole new row (16 elements per lane), so each can quantize it on its own
        const int64_t off = (upd_row * D + dc * EPL) * 2;
        upd_k[0] = load16(mp.k_update, off);
        upd_k[1] = load16(mp.k_update, off + 16);
        upd_v[0] = load16(mp.v_update, off);
        upd_v[1] = load16(mp.v_update, off + 16);
      }
    }
  };
  auto scale_value = [](scale_raw_t raw) -> float {
    if constexpr (SCALE16) {
      return static_cast<float>(__builtin_bit_cast(_Float16, raw));
    } else {
      return raw;
    }
  };

  // Q of a sequence: lane (lr = head, lk) needs dims (D/4)*lk + 8*s + [0, 8) of head h0 + lr, 16 raw bytes per
  // slice for 16-bit queries; fetched when the KV cursor enters the sequence, converted when compute gets there.
  uint4_t qraw[NS];
  // column lr of the MFMA tiles: head lr of the row in a per-row item, (row lr / G, head lr % G) in a shared item
  const int col_seq = GROUPED ? lr / p.group : 0;
  const int col_head = GROUPED ? lr - col_seq * p.group : lr;
  auto issue_q_loads = [&](const TileCursor& c) {
    const bool shared = is_shared(c.b);
    const int m = shared ? col_seq : 0;
    const int g = shared ? col_head : lr;
    const bool live = shared ? m < c.nseq : lr < p.group;
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      qraw[sl] = uint4_t{0u, 0u, 0u, 0u};
      if (live) {
        const int64_t idx =
            (static_cast<int64_t>(c.row + m) * p.q_heads + h0 + g) * DFULL + half * D + (D / 4) * lk + 8 * sl;
        qraw[sl] = load16(p.q, idx * 2);
      }
    }
  };
  V8 qop[NS];
  float qbias = 0.0f;
  auto adopt_q = [&]() {
    float qsum = 0.0f;
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      uint4_t w = qraw[sl];
      if (!q_is_operand_type) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // the other 16-bit float format: go through fp32 (bf16 query with an fp16 operand, or the reverse)
          float a, c;
          if constexpr (KIND == KV_BF16) {
            a = f16_bits_to_float(w[j] & 0xffffu);
            c = f16_bits_to_float(w[j] >> 16);
          } else {
            a = bf16_bits_to_float(w[j] & 0xffffu);
            c = bf16_bits_to_float(w[j] >> 16);
          }
          w[j] = __builtin_bit_cast(uint32_t, make_pair<Pair>(a, c));
        }
      }
      if constexpr (KIND == KV_I8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const Pair pr = __builtin_bit_cast(Pair, static_cast<uint32_t>(w[j]));
          qsum += static_cast<float>(pr.x) + static_cast<float>(pr.y);
        }
      }
      qop[sl] = __builtin_bit_cast(V8, w);
    }
    if constexpr (KIND == KV_I8) qbias = kI8Offset * rows_sum(qsum);
  };

  float4_t acc[NB];
  float m_run = kNegInf, l_run = 0.0f, p_sum = 0.0f;
  auto reset_state = [&]() {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    m_run = kNegInf;
    l_run = 0.0f;
    p_sum = 0.0f;
  };

  auto write_partial = [&](int v, int row, int nseq) {
    // combine the four k-groups' row sums; every lane of a head ends with the head's totals
    const float l_tot = rows_sum(l_run);
    float off = 0.0f;
    if constexpr (KIND == KV_I8) off = kI8Offset * rows_sum(p_sum);
    const bool shared = is_shared(v);
    const bool live = shared ? col_seq < nseq : lr < p.group;
    if (live) {
      // per-row items: slot unit + row, one row per q head; shared items: slot unit + item, 16 columns per kv head
      const int64_t prow = shared ? (static_cast<int64_t>(unit + v) * p.kv_heads + kvh) * 16 + lr
                                  : static_cast<int64_t>(unit + row) * p.q_heads + h0 + lr;
      float* ml = shared ? mp.shared_ml : p.part_ml;
      float* dst = (shared ? mp.shared_acc : p.part_acc) + prow * DFULL + half * D + 4 * lk;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float4_t o = acc[nb];
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = (o[j] - off) * (1.0f / kPScale);
        *reinterpret_cast<float4_t*>(dst + 16 * nb) = o;
      }
      if (lk == 0) {
        ml[prow * 2] = m_run;
        ml[prow * 2 + 1] = l_tot;
      }
    }
  };

  // ---- pair synchronisation of the split-head variant ----------------------------------------------------------------
  int pair_step = 0;  // tiles this wave has gone through; the pair's waves go through the same tiles
  auto pair_wait = [&](const int* flag, int target) {
    // bounded: a partner that never arrives (it cannot, both run the same tile sequence) must not hang the wave
    for (int spin = 0; spin < (1 << 18); ++spin) {
      if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) break;
      __builtin_amdgcn_s_sleep(1);
    }
  };

  // ---- this wave's unit ------------------------------------------------------------------------------------------
  const int bx = blockIdx.x;
  unit = bx < mp.static_wgs ? bx * mp.tok_splits + ts : geo.static_units + (bx - mp.static_wgs) * mp.tok_splits + ts;
  {
    const int x0 = geo.unit_start(unit);
    const int x1 = unit < geo.static_units + geo.small_units ? geo.unit_start(unit + 1) : x0;
    if (x0 < x1) {
      // item that owns tile x0: the largest v with cum[v] <= x0
      int v_first;
      {
        int lo = 0, hi = num_items;
        while (lo + 1 < hi) {
          const int mid = (lo + hi) >> 1;
          if (s_cum[mid] <= x0) {
            lo = mid;
          } else {
            hi = mid;
          }
        }
        v_first = lo;
      }

      // ---- three cursors: block ids are fetched two tiles ahead, KV one tile ahead of the tile being computed ---
      kv_cur.b = v_first;
      enter_item(kv_cur, item_info(v_first));
      kv_cur.next = item_info(v_first + 1);
      kv_cur.tok += (x0 - s_cum[v_first]) * TK;
      id_cur = kv_cur;

      // ---- prologue -------------------------------------------------------------------------------------------
      issue_id_loads();
      issue_q_loads(kv_cur);
      issue_kv_loads();  // tile x0 (waits for its ids)
      if (x0 + 1 < x1) {
        advance(id_cur, x0 + 1);
        issue_id_loads();  // ids of tile x0 + 1
      }
      int cp_b = kv_cur.b, cp_row = kv_cur.row, cp_nseq = kv_cur.nseq, cp_tok = kv_cur.tok, cp_end = kv_cur.end;
      adopt_q();
      reset_state();

      for (int x = x0; x < x1; ++x) {
        ARENO_TRACE_POINT();
        if constexpr (DSPLIT > 1) {
          // the other waves of the head must have read the score part parked in this wave's K tile before the tile
          // is rewritten
#pragma unroll
          for (int part = 0; part < DSPLIT; ++part) {
            if (part != half) pair_wait(&s_pair_flags[1][wave - half + part], pair_step);
          }
        }
        // -- stage the fetched tile into LDS (waits for its loads) ---------------------------------------------
        if (tail_tile) {
          // the newest token: quantize (8-bit caches), substitute it for the unwritten slot, store it into the page
          if constexpr (T::kQuant) {
            uint4_t qk, qv;
            scale_raw_t qks, qvs;
            quantize_row_chunk<KIND, SCALE16, LPT>(upd_k, p.q_dtype, qk, qks);
            quantize_row_chunk<KIND, SCALE16, LPT>(upd_v, p.q_dtype, qv, qvs);
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
              if (cp_tok + i * TPL + grp >= cp_end - 1) {
                kreg[i] = qk;
                vreg[i] = qv;
                ksreg[i] = qks;
                vsreg[i] = qvs;
              }
            }
          }
#pragma unroll
          for (int i = 0; i < NLD; ++i) {
            if (cp_tok + i * TPL + grp == cp_end - 1) {
              char* kc = static_cast<char*>(const_cast<void*>(p.k_cache));
              char* vc = static_cast<char*>(const_cast<void*>(p.v_cache));
              *reinterpret_cast<uint4_t*>(kc + new_row * row_bytes + half_bytes + dc * 16) = kreg[i];
              *reinterpret_cast<uint4_t*>(vc + new_row * row_bytes + half_bytes + dc * 16) = vreg[i];
              if constexpr (T::kQuant) {
                if (dc == 0) {
                  static_cast<scale_raw_t*>(const_cast<void*>(p.k_scale))[new_row] = ksreg[i];
                  static_cast<scale_raw_t*>(const_cast<void*>(p.v_scale))[new_row] = vsreg[i];
                }
              }
            }
          }
        }
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
          const int t = i * TPL + grp;  // tile-local token
          uint4_t kk = kreg[i], vv = vreg[i];
          if constexpr (KIND == KV_I8) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              kk[j] ^= kI8Flip;
              vv[j] ^= kI8Flip;
            }
          }
          *reinterpret_cast<uint4_t*>(k_tile + t * RSK + dc * 16) = kk;
          *reinterpret_cast<uint4_t*>(v_tile + v_row_of(t) * RSV + dc * 16) = vv;
          if (dc == 0) {
            const bool ok = cp_tok + t < cp_end;
            if constexpr (T::kQuant) {
              ksc[t] = ok ? scale_value(ksreg[i]) * p.scale_log2e : kNegInf;
              vsc[t] = ok ? scale_value(vsreg[i]) * kPScale : 0.0f;
            } else {
              ksc[t] = ok ? p.scale_log2e : kNegInf;
              vsc[t] = ok ? kPScale : 0.0f;
            }
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // -- fetch tile x + 1 (its block ids arrived during the previous iteration) and the ids of tile x + 2 ------
        bool next_is_new_seq = false;
        if (x + 1 < x1) {
          next_is_new_seq = advance(kv_cur, x + 1);
          if (next_is_new_seq) issue_q_loads(kv_cur);
          issue_kv_loads();
          if (x + 2 < x1) {
            advance(id_cur, x + 2);
            issue_id_loads();
          }
        }

        // -- S^T = K . Q^T for the two 16-token groups ------------------------------------------------------------
        float s[2][4];
#pragma unroll
        for (int tg = 0; tg < 2; ++tg) {
          float4_t c = {0.0f, 0.0f, 0.0f, 0.0f};
          const char* krow = k_tile + (16 * tg + lr) * RSK + (D / 4) * ES * lk;
          uint32_t kw[NS * WPL];
#pragma unroll
          for (int q4 = 0; q4 < NS * WPL / 4; ++q4) {
            const uint4_t r = *reinterpret_cast<const uint4_t*>(krow + 16 * q4);
            kw[4 * q4 + 0] = r[0];
            kw[4 * q4 + 1] = r[1];
            kw[4 * q4 + 2] = r[2];
            kw[4 * q4 + 3] = r[3];
          }
#pragma unroll
          for (int sl = 0; sl < NS; ++sl) c = Ops::mfma(to_operand<KIND>(&kw[sl * WPL]), qop[sl], c);
          if constexpr (DSPLIT == 1) {
            const float4_t sc = *reinterpret_cast<const float4_t*>(ksc + 16 * tg + 4 * lk);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              // tokens past the end carry a -inf scale; keep them exactly -inf (0 * -inf would be NaN)
              const float v = c[j] - qbias;
              s[tg][j] = sc[j] == kNegInf ? kNegInf : v * sc[j];
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) s[tg][j] = c[j] - qbias;  // this wave's part of the dot products
          }
        }
        if constexpr (DSPLIT > 1) {
          // Park the part where the K tile was (its rows have been read by the products above), tell the other waves of
          // the head, wait for their parts, add all parts in the order of the head dimension.  Every wave of the head
          // ends up with the same eight sums.
          float* mine = reinterpret_cast<float*>(k_tile);
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) mine[(4 * tg + j) * kWave + lane] = s[tg][j];
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          ++pair_step;
          if (lane == 0)
            __hip_atomic_store(&s_pair_flags[0][wave], pair_step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          const int first_wave = wave - half;
          float total[2][4];
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) total[tg][j] = 0.0f;
          }
#pragma unroll
          for (int part = 0; part < DSPLIT; ++part) {
            if (part == half) {
#pragma unroll
              for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) total[tg][j] += s[tg][j];
              }
            } else {
              pair_wait(&s_pair_flags[0][first_wave + part], pair_step);
              __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
              const float* theirs = reinterpret_cast<const float*>(&s_tiles[first_wave + part][0]);
#pragma unroll
              for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
                for (int j = 0; j < 4; ++j) total[tg][j] += theirs[(4 * tg + j) * kWave + lane];
              }
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // the reads above are done before the others hear
          if (lane == 0)
            __hip_atomic_store(&s_pair_flags[1][wave], pair_step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
            const float4_t sc = *reinterpret_cast<const float4_t*>(ksc + 16 * tg + 4 * lk);
#pragma unroll
            for (int j = 0; j < 4; ++j) s[tg][j] = sc[j] == kNegInf ? kNegInf : total[tg][j] * sc[j];
          }
        }

        // -- online softmax for head lr over the tile's 32 tokens ---------------------------------------------------
        float mt = max3_f32(max3_f32(s[0][0], s[0][1], s[0][2]), max3_f32(s[0][3], s[1][0], s[1][1]),
                            max_f32(s[1][2], s[1][3]));
        mt = rows_max(mt);
        const float m_new = max_f32(m_run, mt);
        const float m_safe = m_new == kNegInf ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
          l_run *= alpha;
          p_sum *= alpha;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[nb][j] *= alpha;
          }
        }
        uint32_t pw[4];
        {
          const float4_t vs0 = *reinterpret_cast<const float4_t*>(vsc + 4 * lk);
          const float4_t vs1 = *reinterpret_cast<const float4_t*>(vsc + 16 + 4 * lk);
          float pe[8];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float e0 = fast_exp2(s[0][j] - m_safe);
            const float e1 = fast_exp2(s[1][j] - m_safe);
            l_run += e0 + e1;
            pe[j] = e0 * vs0[j];
            pe[4 + j] = e1 * vs1[j];
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            pw[j] = pack_pair<KIND>(pe[2 * j], pe[2 * j + 1]);
            if constexpr (KIND == KV_I8) {
              const Pair pr = __builtin_bit_cast(Pair, pw[j]);
              p_sum += static_cast<float>(pr.x) + static_cast<float>(pr.y);
            }
          }
        }
        const V8 pop = __builtin_bit_cast(V8, uint4_t{pw[0], pw[1], pw[2], pw[3]});

        // -- O^T += V^T . P^T, one MFMA per 16-dim block -------------------------------------------------------------
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          uint32_t vw[4];
          if constexpr (ES == 1) {
            // lane i of a 16-lane group supplies row (i / 2), 8 bytes at column 16 nb + 8 (i % 2)
            const int r8 = lr >> 1;
            const int tok = r8 < 4 ? 4 * lk + r8 : 16 + 4 * lk + (r8 - 4);
            char* a = v_tile + v_row_of(tok) * RSV + 16 * nb + 8 * (lr & 1);
            const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_int2*)a);
            vw[0] = static_cast<uint32_t>(r[0]);
            vw[1] = static_cast<uint32_t>(r[1]);
          } else {
            // lane i supplies row (i / 4), 4 elements at column 16 nb + 4 (i % 4); two reads of 4 tokens each
            const int r4 = lr >> 2;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              const int tok = 16 * half + 4 * lk + r4;
              char* a = v_tile + v_row_of(tok) * RSV + (16 * nb + 4 * (lr & 3)) * 2;
              const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
              const uint2_t u = __builtin_bit_cast(uint2_t, r);
              vw[2 * half] = u[0];
              vw[2 * half + 1] = u[1];
            }
          }
          acc[nb] = Ops::mfma(to_operand<KIND>(vw), pop, acc[nb]);
        }
        // all LDS reads of this tile are done before the next iteration overwrites it
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // -- end of a sequence's share: emit its partial and switch to the next sequence ---------------------------
        const bool last_of_piece = x + 1 == x1;
        if (next_is_new_seq || last_of_piece) {
          write_partial(cp_b, cp_row, cp_nseq);
          if (!last_of_piece) {
            cp_b = kv_cur.b;
            cp_row = kv_cur.row;
            cp_nseq = kv_cur.nseq;
            adopt_q();
            reset_state();
          }
        }
        cp_tok = kv_cur.tok;
        cp_end = kv_cur.end;
      }
    }
#ifdef ARENO_TRACE
    if (mp.trace && lane == 0) mp.trace[trace_wave * 16 + 1] = wall_clock64();
#endif
  }
}

typedef void (*decode_mfma_fn)(MfmaDecodeParams);
decode_mfma_fn decode_mfma_lookup_bf16(int head_dim, bool scale16, bool grouped);
decode_mfma_fn decode_mfma_lookup_f16(int head_dim, bool scale16, bool grouped);
decode_mfma_fn decode_mfma_lookup_i8(int head_dim, bool scale16, bool grouped);
decode_mfma_fn decode_mfma_lookup_fp8(int head_dim, bool scale16, bool grouped);

template <int KIND, bool GROUPED>
decode_mfma_fn decode_mfma_lookup_impl(int head_dim, bool scale16) {
  constexpr int NW = ARENO_MFMA_NW;
  if constexpr (KVTraits<KIND>::kQuant) {
    if (head_dim == 128)
      return scale16 ? decode_mfma_kernel<KIND, 128, true, NW, GROUPED> : decode_mfma_kernel<KIND, 128, false, NW, GROUPED>;
    if (head_dim == 64)
      return scale16 ? decode_mfma_kernel<KIND, 64, true, NW, GROUPED> : decode_mfma_kernel<KIND, 64, false, NW, GROUPED>;
  } else {
    if (head_dim == 128) return decode_mfma_kernel<KIND, 128, false, NW, GROUPED>;
    if (head_dim == 64) return decode_mfma_kernel<KIND, 64, false, NW, GROUPED>;
  }
  if constexpr (!GROUPED && NW % 2 == 0) {
    // head dim 256: two waves per head, 128 elements each
    if (head_dim == 256) {
      if constexpr (KVTraits<KIND>::kQuant) {
        if (scale16) return decode_mfma_kernel<KIND, 128, true, NW, false, 2>;
      }
      return decode_mfma_kernel<KIND, 128, false, NW, false, 2>;
    }
  }
  if constexpr (!GROUPED && NW % 4 == 0) {
    // head dim 512: four waves per head, 128 elements each
    if (head_dim == 512) {
      if constexpr (KVTraits<KIND>::kQuant) {
        if (scale16) return decode_mfma_kernel<KIND, 128, true, NW, false, 4>;
      }
      return decode_mfma_kernel<KIND, 128, false, NW, false, 4>;
    }
  }
  if constexpr (!GROUPED) {
    // head dim 192: three waves per head, 64 elements each, in workgroups of six waves
    if (head_dim == 192) {
      if constexpr (KVTraits<KIND>::kQuant) {
        if (scale16) return decode_mfma_kernel<KIND, 64, true, 6, false, 3>;
      }
      return decode_mfma_kernel<KIND, 64, false, 6, false, 3>;
    }
  }
  return nullptr;
}

// Waves of a workgroup that share one head (the head-dimension split of decode_mfma_kernel), and the waves per
// workgroup of the kernel the lookup returns for a head dim.
inline int decode_mfma_head_split(int head_dim) {
  return head_dim == 256 ? 2 : (head_dim == 192 ? 3 : (head_dim == 512 ? 4 : 1));
}
inline int decode_mfma_waves(int head_dim) { return head_dim == 192 ? 6 : ARENO_MFMA_NW; }

}  // namespace areno
