// Split-KV GQA paged decode on the matrix cores (gfx950), device code.
//
// Why MFMA for a bandwidth-bound op: at 70 % of 8 TB/s every SIMD must consume ~2.3 KV bytes per clock
// and each int8/fp8 byte needs G = q_heads / kv_heads multiply-adds on the QK^T side and G more on the P.V
// side.  With G = 7 that is more than the vector ALU can issue even with v_dot2, so the VALU kernel
// (paged_decode_kernels.hpp) tops out well below the HBM roofline.  Here the G query heads of one KV head
// form the (zero padded) 16-wide N side of v_mfma_f32_16x16x32 tiles; the vector ALU only dequantizes
// (<= 0.75 op per element) and runs the softmax.
//
// Work decomposition (decode_items.hpp; exactly balanced, no host knowledge of the lengths):
//   * a sequence contributes ceil(visible_keys / 32) tiles of 32 tokens; every workgroup computes the
//     prefix sum of tile counts over the batch in LDS and takes an equal share of the global tile range
//     (a "unit" per wave), so all waves stream the same number of bytes whatever the length distribution;
//   * a unit that crosses a sequence boundary emits one partial per sequence it touches, into slot
//     (unit index + sequence index), which is unique and contiguous per sequence; the reduce kernel merges
//     the slots of each sequence;
//   * block = 4 wave64; wave w owns KV head z*HW + w % HW, so with kv_heads >= 4 the four waves of a
//     workgroup read whole pages ([slot][kv_head][D] is contiguous).  Waves never synchronise after the
//     prefix sum.
// Data path per 32-token tile and wave (lane = (lr, lk) = (lane % 16, lane / 16); token group tg = 0, 1):
//   K  global --16 B/lane--> registers --> MFMA A operand, no LDS: lane (lr, lk) fetches from token 16 tg + lr the
//      16-byte chunks lk, lk + 4, ... of the head's row, i.e. 64 contiguous bytes per token and load instruction.
//      The k index of the products is whatever dims those chunks hold; Q^T (B operand, in registers for the whole
//      sequence) is loaded in the same order, so S^T[token][head] = K . Q^T needs no shuffle.
//   V  global --same lane / chunk assignment--> registers --ds_write_b128--> LDS, chunk-major
//      ([token group][chunk][16 tokens][16 B]; 256 contiguous bytes per 16 lanes) --ds_read_b64_tr_b8 / _tr_b16-->
//      A operand V^T (the LDS transpose read gives each lane 8 tokens of one dim).  So that the 32 lanes of one pass of
//      the transpose read cover all 64 banks once, the second token group starts 128 bytes off a multiple of 256 and,
//      for 16-bit elements (one read touches an even and an odd chunk), an odd chunk keeps its token rows 8..15 in
//      front of rows 0..7.
//   online softmax in the log2 domain on the C layout of S^T (head = lane % 16, 4 tokens per lane and group); the
//      per-token K scale multiplies S, the V scale multiplies P (scales travel through 64 floats of LDS per tile).
//   O^T[dim][head] += V^T . P^T, where P^T *is* the C layout of S^T, so no cross-lane movement of P is needed.
// One tile is in flight per wave: the loads of tile x + 1 go out while tile x is computed (V registers are free once
// the tile is staged, K registers once the scores are issued), the block ids of tile x + 2 in front of them.  The
// loop over the regular tiles of an item has no branches around loads, so every wait the compiler places counts
// exactly the loads younger than the one needed.  Measured on the part: with one workgroup per CU and every wave
// holding a tile in flight the memory system is saturated (an 8 KB tile takes ~1.45 us to arrive, 5.7-5.9 TB/s
// aggregate; with two workgroups per CU 2.6 us), more tiles or waves in flight only lengthen the queues, and fewer
// instructions per step change nothing; what a launch loses is its start (work list, block ids, first tile: ~3.7 us)
// and the spread of the waves' finish times.
// int8 codes become fp16 by placing (code ^ 0x80) under the exponent byte 0x64 (v_perm): 1152 + code exactly;
// the offsets are removed algebraically (1152 * sum(q) per head, 1152 * sum(p) per head).  fp8 uses
// v_cvt_scalef32_pk_f16_fp8 with scale 1 (exact).  bf16 / fp16 caches feed the MFMA directly.
//
// The single-token append (areno/accel/csrc/attention.cu:526-553) rides along as a tile of its own at the end of
// each row's item: the wave that owns it reads the row of k_update / v_update (8 bytes per lane), quantizes it with
// the cache writer's closed form, stores codes and scales into the page and folds the token into its running
// softmax on the vector ALU (one token is not worth a matrix product).  The cached tokens in front of it never touch
// the unwritten slot.  That tile streams nothing: the regular tile in front of it fetches only the update rows, and the
// tile behind it is requested at the start of the token's own step.
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

#include "decode_items.hpp"
#include "paged_decode_kernels.hpp"

namespace areno {

#ifndef ARENO_MFMA_NW
#define ARENO_MFMA_NW 4
#endif
// waves per SIMD the register budget of the 8-bit / 16-bit kernels is set for
#ifndef ARENO_MFMA_QUANT_OCC
#define ARENO_MFMA_QUANT_OCC 2
#endif
#ifndef ARENO_MFMA_WIDE_OCC
#define ARENO_MFMA_WIDE_OCC 2
#endif

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) int int2_t;

struct MfmaDecodeParams {
  DecodeParams d;      // part_ml / part_acc are indexed [slot][q_head] here
  int32_t* plan;       // [items + 1]: exclusive prefix sums of tiles per item (written by workgroup 0)
  int32_t tok_splits;  // waves of a workgroup that share a KV head (waves per workgroup / heads_per_wg / head split)
  int32_t num_units;   // gridDim.x * tok_splits
  ItemShape items;     // rows -> items (prefix groups, window, whether the append rides along)
  // Fused append: per-row items end in a tile for the newest token, whose K / V row comes from here
  // ([batch, kv_heads, head_dim], dtype q_dtype), is quantized like the cache writer does and stored into the page.
  const void* k_update;
  const void* v_update;
  // Prefix groups (GROUPED kernels only): rows [i * group_rows, (i + 1) * group_rows) share the pages of their first
  // shared_lens[i] tokens.  Shared items leave their partials in a second region (16 columns per kv head and slot).
  const int32_t* shared_lens;  // [batch / group_rows]
  float* shared_ml;            // [slot][kv_head][16][2]
  float* shared_acc;           // [slot][kv_head][16][head_dim]
  unsigned long long* trace;   // [wave][8] timestamps; NULL outside tuning runs (ARENO_TRACE builds only read it)
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
  } else if constexpr (KIND == KV_I8) {  // bytes already flipped to offset binary
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

// a wave-uniform value that the compiler cannot prove uniform (it came out of LDS): move it to a scalar register
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// The length arrays and the tile prefix sums in LDS, as the item functions of decode_items.hpp want them.  The
// "uniform" flavour is for lookups whose index is the same in all lanes of a wave (the tile cursors): the values
// then live in scalar registers.
template <bool UNIFORM>
struct LdsLens {
  const int* len;
  const int* glen;
  __device__ __forceinline__ int row_len(int b) const { return UNIFORM ? uniform(len[b]) : len[b]; }
  __device__ __forceinline__ int group_len(int g) const { return UNIFORM ? uniform(glen[g]) : glen[g]; }
};
struct LdsCum {
  const int* cum;
  __device__ __forceinline__ int at(int i) const { return uniform(cum[i]); }
};

// What the pipeline remembers of a tile between the moment its block ids are requested and the moment it is computed
// (all wave-uniform).
struct TileDesc {
  int tok;   // first token of the tile inside its sequence
  int end;   // end of the item's cached tokens
  int row;   // block-table / query row
  int nseq;  // rows side by side (shared items), else 1
  int b;     // item index
  int x_end; // global index of the item's last tile + 1
  int kind;  // bit 0: the tile opens its item; bit 1: it holds only the token being appended; bit 2: past the unit
};
constexpr int kTileOpens = 1, kTileNewToken = 2, kTilePhantom = 4;

// DSPLIT > 1 serves heads of DSPLIT * D elements (256 = 2 x 128, 192 = 3 x 64, 512 = 4 x 128): DSPLIT adjacent waves
// of the workgroup take one part of the head dimension each.  Every wave computes the part of S = K . Q^T over its
// elements, the waves exchange the parts through LDS, add them in the same order and go on with identical scores:
// the same softmax in all, P . V over the wave's own part of V, the wave's part of the partial row.  The waves of a
// head synchronise through two counters each in LDS (part ready / parts consumed); no workgroup barrier is involved,
// so the heads of one workgroup may run different units.
template <int KIND, int D, bool SCALE16, int NW, bool GROUPED = false, int DSPLIT = 1>
__global__ __launch_bounds__(NW * kWave, KVTraits<KIND>::kQuant ? ARENO_MFMA_QUANT_OCC : ARENO_MFMA_WIDE_OCC) void decode_mfma_kernel(
    MfmaDecodeParams mp) {
  using T = KVTraits<KIND>;
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using Pair = typename T::pair_t;
  const DecodeParams& p = mp.d;
  constexpr int ES = T::kBytes;
  constexpr int TK = kTileTokens;
  constexpr int CPT = D * ES / 16;     // 16-byte chunks per token row
  constexpr int CPL = CPT / 4;         // chunks per lane and token: lk, lk + 4, ...
  constexpr int NS = D / 32;           // QK^T k-slices
  constexpr int NB = D / 16;           // P.V dim blocks
  constexpr int WPS = 8 * ES / 4;      // dwords per k-slice of 8 elements
  constexpr int TGS = CPT * 256 + 128;    // bytes of one token group of the V tile in LDS (128 of padding behind it)
  constexpr float kPScale = T::kQuant ? 256.0f : 1.0f;
  constexpr int kParkFloats = DSPLIT > 1 ? 8 * kWave : 0;
  constexpr int kWaveLds = 2 * TGS + 2 * TK * 4 + kParkFloats * 4;
  constexpr int UPW = D / 64;          // dwords per lane of an update row pair (K row in lanes 0..31, V row in 32..63)
  static_assert(CPL >= 1 && CPL <= 4 && (D == 64 || D == 128), "unsupported head_dim");
  static_assert(2 * TGS >= 2 * D * 4, "the new token's rows borrow the V tile");
  static_assert(DSPLIT == 1 || (DSPLIT >= 2 && DSPLIT <= 4 && !GROUPED && NW % DSPLIT == 0), "unsupported head split");
  constexpr int DFULL = D * DSPLIT;  // elements of a whole head (row of Q, of a cache page, of a partial)

  __shared__ __attribute__((aligned(16))) char s_tiles[NW][kWaveLds];
  constexpr int kMaxItems = (GROUPED ? 2 : 1) * kMfmaMaxBatch;  // at most one shared item per row on top of the rows
  __shared__ int s_cum[kMaxItems + 1];
  __shared__ int s_wave_tot[NW];
  __shared__ int s_len[kMfmaMaxBatch];                          // sequence lengths of the rows
  constexpr int kMaxGroups = kMfmaMaxBatch / 2;                 // groups have at least two rows
  __shared__ int s_group_len[GROUPED ? kMaxGroups : 1];         // shared prefix length of each group
  __shared__ int s_pair_flags[2][NW];  // [0]: score parts this wave has published, [1]: steps whose parts it has read
  constexpr int SPT = (kMaxItems + NW * kWave - 1) / (NW * kWave);  // items per thread in the prefix sum

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: the unit's bounds and the loop follow
#ifdef ARENO_TRACE
  const int trace_wave = (blockIdx.y * gridDim.x + blockIdx.x) * NW + wave;
  int trace_n = 1;
  if (mp.trace && lane == 0) {
    // start time, and in word 7 where the wave runs: XCC id (hardware register 20) above the HW_ID word (register 4)
    mp.trace[trace_wave * 8] = wall_clock64();
    mp.trace[trace_wave * 8 + 7] = (static_cast<unsigned long long>(__builtin_amdgcn_s_getreg((31 << 11) | 20)) << 32) |
                                    static_cast<unsigned int>(__builtin_amdgcn_s_getreg((31 << 11) | 4));
  }
#define ARENO_TRACE_POINT() \
  if (mp.trace && lane == 0 && trace_n < 6) mp.trace[trace_wave * 8 + trace_n++] = wall_clock64()
#else
#define ARENO_TRACE_POINT()
#endif
  const int lr = lane & 15;  // MFMA row / column index
  const int lk = lane >> 4;  // MFMA k group

  // ---- the item list: lengths into LDS, tiles per item, exclusive prefix sum over the items ------------------------
  const ItemShape& shape = mp.items;
  const int num_items = shape.num_items();
  const LdsLens<false> lens_any = {s_len, s_group_len};
  const LdsLens<true> lens = {s_len, s_group_len};
  const LdsCum cum = {s_cum};
  {
    int nt[SPT];
    int local = 0;
    if constexpr (GROUPED) {
      // an item's extent takes the group's length, its members' lengths and the row's own: the workgroup copies both
      // arrays with independent loads first (the launcher sends at most kMfmaMaxBatch rows in groups of >= 2)
      for (int i = tid; i < shape.batch; i += NW * kWave) s_len[i] = p.cache_seqlens[i];
      for (int i = tid; i < shape.num_groups(); i += NW * kWave) s_group_len[i] = mp.shared_lens[i];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        nt[j] = v < num_items ? item_info<true>(shape, lens_any, v).tiles() : 0;
        local += nt[j];
      }
    } else {
      // the thread's sequence lengths are fetched together (clamped index, no branch around the load)
      int len[SPT];
#pragma unroll
      for (int j = 0; j < SPT; ++j) len[j] = p.cache_seqlens[min(SPT * tid + j, num_items - 1)];
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        nt[j] = 0;
        if (v < num_items) {
          s_len[v] = len[j];
          ItemInfo it;
          it.lo = first_visible_key(len[j] + 1, shape.window_left);
          it.end = len[j] + 1 - shape.new_token_tile;
          it.has_new = shape.new_token_tile;
          nt[j] = it.tiles();
        }
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
  const int total_tiles = cum.at(num_items);
  const UnitGeometry geo = make_unit_geometry(total_tiles, mp.num_units);
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    for (int v = tid; v <= num_items; v += NW * kWave) mp.plan[v] = s_cum[v];
  }
  ARENO_TRACE_POINT();

  const int hw_count = p.heads_per_wg;
  const int half = wave % DSPLIT;  // which part of the head dimension this wave owns
  const int hw = (wave / DSPLIT) % hw_count;
  const int ts = (wave / DSPLIT) / hw_count;
  const int kvh = blockIdx.y * hw_count + hw;
  char* const v_tile = &s_tiles[wave][0];
  float* const sc_lds = reinterpret_cast<float*>(&s_tiles[wave][2 * TGS]);  // [0, 32): K scales, [32, 64): V scales
  float* const park = reinterpret_cast<float*>(&s_tiles[wave][2 * TGS + 2 * TK * 4]);

  constexpr int64_t row_bytes = static_cast<int64_t>(DFULL) * ES;
  const int64_t half_bytes = static_cast<int64_t>(half) * D * ES;  // of this wave's part inside a cache / update row
  const int h0 = kvh * p.group;
  const bool q_is_operand_type = (KIND == KV_BF16 && p.q_dtype == ARENO_DT_BF16) ||
                                 (KIND != KV_BF16 && p.q_dtype == ARENO_DT_F16);
  auto is_shared = [&](int v) { return GROUPED && v < shape.num_shared; };
  // first element of the 8 that k-slice sl holds in this lane (the chunk order of the K loads)
  auto slice_base = [&](int sl) { return ES == 1 ? 16 * (lk + 4 * (sl >> 1)) + 8 * (sl & 1) : 8 * (lk + 4 * sl); };
  // byte offset of token row r (0..15) of chunk c inside a token group of the V tile: 16-bit tiles keep the two
  // halves of an odd chunk's rows swapped (see the layout note above)
  auto chunk_row_pos = [](int c, int r) { return c * 256 + ((ES == 2 && (c & 1)) ? (r ^ 8) : r) * 16; };

  // ---- the pipeline's registers ------------------------------------------------------------------------------------
  // Every step issues the same loads in the same order whatever the kinds of the tiles involved (only their addresses
  // differ), so that the waits the compiler places count exactly the loads that are younger than the one needed and
  // the tiles behind it stay in flight.  Loads that depend on a tile's kind (the update rows of an appended token, the
  // Q of the next item) are extra loads on rare paths.
  typedef typename std::conditional<SCALE16, uint16_t, float>::type scale_raw_t;
  uint4_t kreg[2 * CPL], vreg[2 * CPL];
  scale_raw_t sreg;   // lane l < 32: K scale of tile token l; else V scale of token l - 32
  uint32_t upd[UPW];  // a new-token tile: the update rows, K in lanes 0..31, V in 32..63
  uint32_t new_row = 0;   // a new-token tile: cache row (block, slot, head) the token goes to
  TileDesc desc0;      // the tile whose loads are in the registers
  TileCursor cur;      // the furthest tile requested so far (its block ids are on their way)
  TileDesc desc_ids;   // = that tile

  auto describe = [&](const TileCursor& c, bool opens) {
    TileDesc t;
    t.tok = c.tok;
    t.end = c.it.end;
    t.row = c.it.row;
    t.nseq = c.it.nseq;
    t.b = c.b;
    t.x_end = c.x_end;
    t.kind = (opens ? kTileOpens : 0) | (c.on_new_token() ? kTileNewToken : 0);
    return t;
  };
  // (the launcher sends only page sizes that are powers of two here)
  auto column_of = [&](int t) { return t >> p.bs_shift; };
  auto slot_of = [&](int t) { return t & (p.block_size - 1); };
  // The token whose cache row this lane fetches for group tg: its own token of a regular tile (clamped to the last
  // cached one); the position being appended for a new-token tile (the row is not used, it only has to exist); one
  // token for all lanes of a phantom tile (a tile past the unit's end: its loads keep the pipeline's shape and hit
  // one cache line each).
  auto lane_token = [&](const TileDesc& t, int tg) {
    const int own = (t.kind & kTilePhantom) ? 0 : 16 * tg + lr;
    return (t.kind & kTileNewToken) ? t.end : min(t.tok + own, t.end - 1);
  };
  // (block ids and cache rows are pairs of scalars, one per token group, not arrays: an array indexed by a lane-dependent
  // value would live in scratch memory, and scratch loads count with the global loads and drain the pipeline)
  struct IdPair {
    int g0, g1;
  };
  auto issue_id_loads = [&](const TileDesc& t) {
    const int32_t* table_row = p.block_table + static_cast<int64_t>(t.row) * p.max_blocks;
    IdPair r;
    r.g0 = table_row[column_of(lane_token(t, 0))];
    r.g1 = table_row[column_of(lane_token(t, 1))];
    return r;
  };
  // cache row (block, slot, head) of this lane's token of each group, from the block ids that have arrived
  uint32_t row_g0 = 0, row_g1 = 0;
  auto rows_from_ids = [&](const TileDesc& t, const IdPair& src) {
    row_g0 = (static_cast<uint32_t>(src.g0) * p.block_size + slot_of(lane_token(t, 0))) * p.kv_heads + kvh;
    row_g1 = (static_cast<uint32_t>(src.g1) * p.block_size + slot_of(lane_token(t, 1))) * p.kv_heads + kvh;
  };
  // what an appended token's tile needs: the update rows (first 32 lanes K, the others V) and the cache row they go to
  auto issue_update_loads = [&](const TileDesc& t) {
    if constexpr (DSPLIT == 1) {
      if ((t.kind & (kTileNewToken | kTilePhantom)) == kTileNewToken) {
        const void* src = lane < 32 ? mp.k_update : mp.v_update;
        const int64_t off = (static_cast<int64_t>(t.row) * p.kv_heads + kvh) * D * 2 + (lane & 31) * (UPW * 4);
#pragma unroll
        for (int w = 0; w < UPW; ++w) upd[w] = *reinterpret_cast<const uint32_t*>(static_cast<const char*>(src) + off + 4 * w);
      }
      new_row = row_g0;
    }
  };
  auto issue_v_loads = [&](const TileDesc& t) {
    issue_update_loads(t);
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      const char* va = static_cast<const char*>(p.v_cache) + (tg ? row_g1 : row_g0) * row_bytes + half_bytes + lk * 16;
#pragma unroll
      for (int j = 0; j < CPL; ++j) vreg[tg * CPL + j] = *reinterpret_cast<const uint4_t*>(va + 64 * j);
    }
    if constexpr (T::kQuant) {
      const uint32_t r = (lk & 1) ? row_g1 : row_g0;
      const void* sp = lk < 2 ? p.k_scale : p.v_scale;
      sreg = static_cast<const scale_raw_t*>(sp)[r];
    }
  };
  auto issue_k_loads = [&](const TileDesc& t) {
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      const char* ka = static_cast<const char*>(p.k_cache) + (tg ? row_g1 : row_g0) * row_bytes + half_bytes + lk * 16;
#pragma unroll
      for (int j = 0; j < CPL; ++j) kreg[tg * CPL + j] = *reinterpret_cast<const uint4_t*>(ka + 64 * j);
    }
  };
  auto scale_value = [](scale_raw_t raw) -> float {
    if constexpr (SCALE16) {
      return static_cast<float>(__builtin_bit_cast(_Float16, raw));
    } else {
      return raw;
    }
  };

  // Q of an item: lane (lr = column, lk) needs, per k-slice, the 8 elements the K loads put there; 16 raw bytes per
  // slice for 16-bit queries.  Requested one step before the item's first tile is computed, converted when compute
  // gets there.  Column lr of the MFMA tiles: head lr of the row in a per-row item, (row lr / G, head lr % G) in a
  // shared item.
  uint4_t qraw[NS];
  const int col_seq = GROUPED ? lr / p.group : 0;
  const int col_head = GROUPED ? lr - col_seq * p.group : lr;
  auto issue_q_loads = [&](int item, int row, int nseq) {
    const bool shared = is_shared(item);
    const int m = shared ? col_seq : 0;
    const int g = shared ? col_head : lr;
    const bool live = shared ? m < nseq : lr < p.group;
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      qraw[sl] = uint4_t{0u, 0u, 0u, 0u};
      if (live) {
        const int64_t idx = (static_cast<int64_t>(row + m) * p.q_heads + h0 + g) * DFULL + half * D + slice_base(sl);
        qraw[sl] = load16(p.q, idx * 2);
      }
    }
  };
  V8 qop[NS];
  float qbias = 0.0f;
  float4_t score_init = {0.0f, 0.0f, 0.0f, 0.0f};  // what the score products accumulate onto: -qbias for int8, else 0
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
    if constexpr (KIND == KV_I8) {
      qbias = kI8Offset * rows_sum(qsum);
      score_init = float4_t{-qbias, -qbias, -qbias, -qbias};
    }
  };

  float4_t acc[NB];
  float m_run = kNegInf, l_run = 0.0f;
  // int8: sum over the item's tokens of the probabilities as rounded for P . V, which the offset of the V operands is
  // taken out with; from the matrix cores (an all-ones A operand puts the column's sum over the tile's 32 tokens, all
  // four k groups included, into every element), like the products it corrects
  float4_t p_sum = {0.0f, 0.0f, 0.0f, 0.0f};
  auto reset_state = [&]() {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    m_run = kNegInf;
    l_run = 0.0f;
    p_sum = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  };

  int unit = 0;
  auto write_partial = [&](int v, int row, int nseq) {
    // combine the four k-groups' row sums; every lane of a head ends with the head's totals
    const float l_tot = rows_sum(l_run);
    float off = 0.0f;
    if constexpr (KIND == KV_I8) off = kI8Offset * p_sum[0];
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
  auto lds_fence = [&]() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // ---- the token being appended: quantize, store into the page, fold into the running softmax (vector ALU) ---------
  // `after_read` runs once the update rows are out of their load registers: the next tile's loads go out there, ahead
  // of the arithmetic, which is long for a step that streams nothing (the next tile may be an appended token's as well
  // and load into the same registers).
  auto new_token_step = [&](const TileDesc& t, auto&& after_read) {
    if constexpr (DSPLIT == 1) {
      constexpr int EPU = 2 * UPW;  // elements of the row this lane holds: (lane % 32) * EPU ...
      const int sub = lane & 31;
      const bool is_v = lane >= 32;
      float x[EPU];
      uint32_t raw_row[UPW];
#pragma unroll
      for (int w = 0; w < UPW; ++w) raw_row[w] = upd[w];
      const int64_t dst_row = new_row;  // (the loads of the next tile replace it with theirs)
      after_read();
#pragma unroll
      for (int w = 0; w < UPW; ++w) {
        const uint32_t word = raw_row[w];
        if (p.q_dtype == ARENO_DT_BF16) {
          x[2 * w] = bf16_bits_to_float(word & 0xffffu);
          x[2 * w + 1] = bf16_bits_to_float(word >> 16);
        } else {
          x[2 * w] = f16_bits_to_float(word & 0xffffu);
          x[2 * w + 1] = f16_bits_to_float(word >> 16);
        }
      }
      char* cache = static_cast<char*>(const_cast<void*>(is_v ? p.v_cache : p.k_cache));
      float xhat[EPU];  // what a reader of the page sees
      if constexpr (T::kQuant) {
        float amax = 0.0f;
#pragma unroll
        for (int e = 0; e < EPU; ++e) amax = fmaxf(amax, fabsf(x[e]));
#pragma unroll
        for (int m = 1; m < 32; m <<= 1) amax = fmaxf(amax, wave_xor(amax, m));
        float s, s_stored;
        scale_raw_t raw;
        if constexpr (KIND == KV_I8) {
          const _Float16 s16 = static_cast<_Float16>(fminf(amax / 127.0f, 65504.0f));
          const _Float16 s16_fixed = (s16 == static_cast<_Float16>(0.0f)) ? static_cast<_Float16>(1.0f) : s16;
          s = static_cast<float>(s16_fixed);
          s_stored = s;
          if constexpr (SCALE16) {
            raw = __builtin_bit_cast(uint16_t, s16_fixed);
          } else {
            raw = s;
          }
        } else {
          s = amax / 448.0f;
          if (s == 0.0f) s = 1.0f;
          if constexpr (SCALE16) {
            raw = static_cast<uint16_t>(float_to_f16_bits(s));
            s_stored = f16_bits_to_float(raw);
          } else {
            raw = s;
            s_stored = s;
          }
        }
        uint32_t word = 0;
#pragma unroll
        for (int e = 0; e < EPU; ++e) {
          uint32_t byte;
          float code_value;
          if constexpr (KIND == KV_I8) {
            const float code = fminf(fmaxf(rintf(x[e] / s), -127.0f), 127.0f);
            byte = static_cast<uint32_t>(static_cast<int>(code)) & 0xffu;
            code_value = code;
          } else {
            byte = float_to_fp8_byte(fminf(fmaxf(x[e] / s, -448.0f), 448.0f));
            code_value = fp8_byte_to_float(byte);
          }
          word |= byte << (8 * e);
          xhat[e] = code_value * s_stored;
        }
        char* dst = cache + dst_row * row_bytes + sub * EPU;
        if constexpr (EPU == 4) {
          *reinterpret_cast<uint32_t*>(dst) = word;
        } else {
          *reinterpret_cast<uint16_t*>(dst) = static_cast<uint16_t>(word);
        }
        if (sub == 0) static_cast<scale_raw_t*>(const_cast<void*>(is_v ? p.v_scale : p.k_scale))[dst_row] = raw;
      } else {
        // 16-bit pages hold the update row as it is (the launcher only fuses when the dtypes agree)
        char* dst = cache + dst_row * row_bytes + sub * (EPU * 2);
#pragma unroll
        for (int w = 0; w < UPW; ++w) *reinterpret_cast<uint32_t*>(dst + 4 * w) = raw_row[w];
#pragma unroll
        for (int e = 0; e < EPU; ++e) xhat[e] = x[e];
      }
      // both rows as floats where the V tile is (no tile is staged at this point): K row, then V row
      float* rowbuf = reinterpret_cast<float*>(v_tile);
#pragma unroll
      for (int e = 0; e < EPU; ++e) rowbuf[(is_v ? D : 0) + sub * EPU + e] = xhat[e];
      lds_fence();
      // score of the token for column lr: this lane's 8 elements of every k-slice, then the four lanes of the column
      float dot = 0.0f;
#pragma unroll
      for (int sl = 0; sl < NS; ++sl) {
        const float* kk = rowbuf + slice_base(sl);
        const uint4_t qw = __builtin_bit_cast(uint4_t, qop[sl]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const Pair pr = __builtin_bit_cast(Pair, static_cast<uint32_t>(qw[j]));
          dot += static_cast<float>(pr.x) * kk[2 * j] + static_cast<float>(pr.y) * kk[2 * j + 1];
        }
      }
      const float s_new = rows_sum(dot) * p.scale_log2e;
      const float m_new = max_f32(m_run, s_new);
      const float alpha = fast_exp2(m_run - m_new);  // m_run = -inf for a row without cached tokens -> 0
      const float pn = fast_exp2(s_new - m_new);
      m_run = m_new;
      l_run = l_run * alpha + (lk == 0 ? pn : 0.0f);
#pragma unroll
      for (int j = 0; j < 4; ++j) p_sum[j] *= alpha;
      const float pv = pn * kPScale;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const float4_t vv = *reinterpret_cast<const float4_t*>(rowbuf + D + 16 * nb + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[nb][j] = acc[nb][j] * alpha + pv * vv[j];
      }
      lds_fence();
    } else {
      after_read();  // (the split-head variant appends in a launch of its own and never gets here)
    }
  };

  // ---- one regular tile: stage V and the scales, scores, softmax, P.V ----------------------------------------------
  // `between_v` runs once the V registers of the set are free, `between_k` once the K registers are.
  auto tile_step = [&](const TileDesc& t, auto&& between_v, auto&& between_k) {
    if constexpr (DSPLIT > 1) {
      // the other waves of the head must have read the score part this wave parked in the previous step
#pragma unroll
      for (int part = 0; part < DSPLIT; ++part) {
        if (part != half) pair_wait(&s_pair_flags[1][wave - half + part], pair_step);
      }
    }
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        uint4_t vv = vreg[tg * CPL + j];
        if constexpr (KIND == KV_I8) {
#pragma unroll
          for (int w = 0; w < 4; ++w) vv[w] ^= kI8Flip;
        }
        *reinterpret_cast<uint4_t*>(v_tile + tg * TGS + chunk_row_pos(lk + 4 * j, lr)) = vv;
      }
    }
    if constexpr (T::kQuant) {
      const bool ok = t.tok + (lane & 31) < t.end;
      const float s = scale_value(sreg);
      sc_lds[lane] = lane < 32 ? (ok ? s * p.scale_log2e : kNegInf) : (ok ? s * kPScale : 0.0f);
    }
    lds_fence();
    between_v();  // the V registers of the set are free

    // -- S^T = K . Q^T for the two 16-token groups ------------------------------------------------------------------
    float s[2][4];
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      // int8: the products start from -1152 * sum(q) (score_init), which takes the offset of the operands out again
      float4_t c = score_init;
#pragma unroll
      for (int sl = 0; sl < NS; ++sl) {
        uint32_t w[WPS];
#pragma unroll
        for (int i = 0; i < WPS; ++i) {
          const int word = sl * WPS + i;  // dword of this lane's row part, in load order
          w[i] = kreg[tg * CPL + word / 4][word % 4];
          if constexpr (KIND == KV_I8) w[i] ^= kI8Flip;
        }
        c = Ops::mfma(to_operand<KIND>(w), qop[sl], c);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) s[tg][j] = c[j];  // (this wave's part of) the dot products
    }
    between_k();
    if constexpr (DSPLIT > 1) {
      // Park the part, tell the other waves of the head, wait for their parts, add all parts in the order of the head
      // dimension.  Every wave of the head ends up with the same eight sums.
#pragma unroll
      for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
        for (int j = 0; j < 4; ++j) park[(4 * tg + j) * kWave + lane] = s[tg][j];
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
          const float* theirs = reinterpret_cast<const float*>(&s_tiles[first_wave + part][2 * TGS + 2 * TK * 4]);
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
#pragma unroll
        for (int j = 0; j < 4; ++j) s[tg][j] = total[tg][j];
      }
    }
    // the per-token K scale (softmax scale and log2 e folded in); tokens past the end become exactly -inf, which only
    // an item's last tile has: every other tile takes the branch with one multiply per score
    float vs[2][4];
    const bool whole_tile = t.tok + TK <= t.end;  // (scalar)
#pragma unroll
    for (int tg = 0; tg < 2; ++tg) {
      if constexpr (T::kQuant) {
        const float4_t vv = *reinterpret_cast<const float4_t*>(sc_lds + 32 + 16 * tg + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) vs[tg][j] = vv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) vs[tg][j] = 1.0f;
      }
    }
    if (whole_tile) {
#pragma unroll
      for (int tg = 0; tg < 2; ++tg) {
        float4_t ks = {p.scale_log2e, p.scale_log2e, p.scale_log2e, p.scale_log2e};
        if constexpr (T::kQuant) ks = *reinterpret_cast<const float4_t*>(sc_lds + 16 * tg + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) s[tg][j] *= ks[j];
      }
    } else {
#pragma unroll
      for (int tg = 0; tg < 2; ++tg) {
        if constexpr (T::kQuant) {
          const float4_t ks = *reinterpret_cast<const float4_t*>(sc_lds + 16 * tg + 4 * lk);
#pragma unroll
          for (int j = 0; j < 4; ++j) s[tg][j] = ks[j] == kNegInf ? kNegInf : s[tg][j] * ks[j];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bool ok = t.tok + 16 * tg + 4 * lk + j < t.end;
            s[tg][j] = ok ? s[tg][j] * p.scale_log2e : kNegInf;
          }
        }
      }
    }

    // -- online softmax for column lr over the tile's 32 tokens ------------------------------------------------------
    float mt = max3_f32(max3_f32(s[0][0], s[0][1], s[0][2]), max3_f32(s[0][3], s[1][0], s[1][1]),
                        max_f32(s[1][2], s[1][3]));
    mt = rows_max(mt);
    const float m_new = max_f32(m_run, mt);
    const float m_safe = m_new == kNegInf ? 0.0f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
      l_run *= alpha;
#pragma unroll
      for (int j = 0; j < 4; ++j) p_sum[j] *= alpha;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[nb][j] *= alpha;
      }
    }
    uint32_t pw[4];
    {
      float pe[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e0 = fast_exp2(s[0][j] - m_safe);
        const float e1 = fast_exp2(s[1][j] - m_safe);
        l_run += e0 + e1;
        pe[j] = T::kQuant ? e0 * vs[0][j] : e0;
        pe[4 + j] = T::kQuant ? e1 * vs[1][j] : e1;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pw[j] = pack_pair<KIND>(pe[2 * j], pe[2 * j + 1]);
      }
    }
    const V8 pop = __builtin_bit_cast(V8, uint4_t{pw[0], pw[1], pw[2], pw[3]});
    if constexpr (KIND == KV_I8) {
      constexpr uint32_t kOnes = 0x3c003c00u;  // two fp16 1.0
      p_sum = Ops::mfma(__builtin_bit_cast(V8, uint4_t{kOnes, kOnes, kOnes, kOnes}), pop, p_sum);
    }

    // -- O^T += V^T . P^T, one MFMA per 16-dim block -----------------------------------------------------------------
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      uint32_t vw[4];
      if constexpr (ES == 1) {
        // lane i of a 16-lane group supplies token row (i / 2), 8 bytes at column 8 (i % 2) of chunk nb: rows 0..3 are
        // tokens 4 lk .. 4 lk + 3 of group 0, rows 4..7 the same tokens of group 1
        const int r8 = lr >> 1;
        const int tg = r8 >> 2;
        const int tok = 4 * lk + (r8 & 3);
        char* a = v_tile + tg * TGS + chunk_row_pos(nb, tok) + 8 * (lr & 1);
        const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_int2*)a);
        vw[0] = static_cast<uint32_t>(r[0]);
        vw[1] = static_cast<uint32_t>(r[1]);
      } else {
        // lane i supplies token row (i / 4), 4 elements at column 4 (i % 4) of the 16-dim block: chunk 2 nb + (i % 4) / 2,
        // byte 8 ((i % 4) % 2); two reads of 4 tokens, one per token group
        const int r4 = lr >> 2;
        const int c4 = lr & 3;
#pragma unroll
        for (int tg = 0; tg < 2; ++tg) {
          char* a = v_tile + tg * TGS + chunk_row_pos(2 * nb + (c4 >> 1), 4 * lk + r4) + 8 * (c4 & 1);
          const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
          const uint2_t u = __builtin_bit_cast(uint2_t, r);
          vw[2 * tg] = u[0];
          vw[2 * tg + 1] = u[1];
        }
      }
      acc[nb] = Ops::mfma(to_operand<KIND>(vw), pop, acc[nb]);
    }
    // all LDS reads of this tile are done before the next step overwrites it
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- this wave's unit --------------------------------------------------------------------------------------------
  unit = blockIdx.x * mp.tok_splits + ts;
  const int x0 = geo.unit_start(unit);
  const int x1 = geo.unit_start(unit + 1);
  if (x0 < x1) {
    // move the request cursor to tile x (a phantom past the unit's end) and ask for its block ids
    IdPair ids;  // block ids of the tile the request cursor is on
    auto request = [&](int x) {
      if (x < x1) {
        const bool opens = cursor_advance<GROUPED>(cur, shape, lens, cum, x);
        desc_ids = describe(cur, opens);
      } else {
        desc_ids.kind = (desc_ids.kind & kTileNewToken) | kTilePhantom;
      }
      ids = issue_id_loads(desc_ids);
    };
    // ---- prologue: block ids of the first two tiles one behind the other, Q of the first item, the first tile's
    // loads ------------------------------------------------------------------------------------------------------------
    cursor_seek<GROUPED>(cur, shape, lens, cum, x0);
    desc_ids = describe(cur, true);
    const IdPair ids_first = issue_id_loads(desc_ids);
    issue_q_loads(desc_ids.b, desc_ids.row, desc_ids.nseq);
    desc0 = desc_ids;
    request(x0 + 1);
    rows_from_ids(desc0, ids_first);
    issue_v_loads(desc0);
    issue_k_loads(desc0);
    adopt_q();
    reset_state();

    // One step of the pipeline on the tile in the registers (tile x): the ids of tile x + 1 have arrived (requested a
    // step ago), those of tile x + 2 are requested, and tile x + 1's loads go out as `work` frees the V registers
    // (`between_v`) and the K registers (`between_k`).
    auto step = [&](int x, auto&& work, auto stream_next) {
      ARENO_TRACE_POINT();
      const TileDesc t = desc0;
      const TileDesc nt = desc_ids;
      rows_from_ids(nt, ids);
      // the ids are consumed before the next ones are requested into the same registers
      __builtin_amdgcn_sched_barrier(0);
      request(x + 2);
      // (scheduling barriers: a load of the next tile must not move in front of the last use of the registers it
      // fills, or the two values would need different registers and a copy of a value still in flight)
      work(
          t,
          [&]() {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(stream_next)::value) {
              issue_v_loads(nt);
            } else {
              issue_update_loads(nt);  // the next tile is an appended token's: it streams nothing
            }
            __builtin_amdgcn_sched_barrier(0);
          },
          [&]() {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (decltype(stream_next)::value) issue_k_loads(nt);
            __builtin_amdgcn_sched_barrier(0);
          });
      desc0 = nt;
    };
    using std::false_type;
    using std::true_type;

    // The unit as a sequence of item segments: the tiles of one item that fall into the unit.  The loop over a
    // segment's regular tiles has no item logic in it (so nothing but the tile stream is carried around it); the
    // appended token's tile, the partial and the switch to the next item's Q come behind it.
    int x = x0;
    for (;;) {
      const TileDesc first = desc0;
      const int seg_end = min(x1, first.x_end);
      const bool appended = shape.new_token_tile && !is_shared(first.b) && seg_end == first.x_end;
      const int regular_end = seg_end - (appended ? 1 : 0);
      if (first.x_end < x1) {
        // Q of the next item with tiles: requested now (qraw is free), adopted when this segment is done
        int b2 = first.b + 1;
        while (cum.at(b2 + 1) == first.x_end) ++b2;
        const ItemInfo it2 = item_info<GROUPED>(shape, lens, b2);
        issue_q_loads(b2, it2.row, it2.nseq);
      }
      // An appended token's tile streams nothing, so the regular tile in front of it fetches only the update rows,
      // and the tile behind it is requested at the start of the appended token's own step.
      auto regular = [&](const TileDesc& t, auto&& between_v, auto&& between_k) { tile_step(t, between_v, between_k); };
      const int streaming_end = regular_end - (appended ? 1 : 0);
      for (; x < streaming_end; ++x) step(x, regular, true_type{});
      if (appended) {
        if (x < regular_end) {
          step(x, regular, false_type{});
          ++x;
        }
        step(
            x,
            [&](const TileDesc& t, auto&& between_v, auto&& between_k) {
              new_token_step(t, [&]() {
                between_v();
                between_k();
              });
            },
            true_type{});
        ++x;
      }
      write_partial(first.b, first.row, first.nseq);
      if (x >= x1) break;
      adopt_q();
      reset_state();
    }
  }
#ifdef ARENO_TRACE
  if (mp.trace && lane == 0) mp.trace[trace_wave * 8 + 6] = wall_clock64();
#endif
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
