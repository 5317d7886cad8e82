// Split-KV GQA paged decode on the matrix cores (gfx950), device code.
//
// Why MFMA for a bandwidth-bound op: at 70 % of 8 TB/s every SIMD must consume ~2.3 KV bytes per clock
// and each int8/fp8 byte needs G = q_heads / kv_heads multiply-adds on the QK^T side and G more on the P.V
// side.  With G = 7 that is more than the vector ALU can issue even with v_dot2, so the VALU kernel
// (paged_decode_kernels.hpp) tops out well below the HBM roofline.  Here the G query heads of one KV head
// form the (zero padded) 16-wide N side of v_mfma_f32_16x16x32 tiles; the vector ALU only dequantizes
// (<= 0.75 op per element) and runs the softmax.
//
// Work decomposition (decode_items.hpp; balanced to within 16 tokens, no host knowledge of the lengths):
//   * a sequence contributes ceil(visible cached keys / 16) quanta; the quanta of all sequences are cut into equal
//     ranges, one "unit" per wave, so all waves stream the same number of bytes whatever the length distribution;
//     a wave walks its unit in tile steps of TK tokens (32; the step is generic in TK, and 64-token steps for 8-bit
//     pages, 16 KB in flight per wave like a 16-bit tile, measured slower), the last step of a segment masked;
//   * the list of items (first token, end, row) and the prefix sums of their quanta live in LDS: every workgroup
//     computes them from the sequence lengths, or copies them from a plan that areno_hip_paged_decode_plan left in
//     device memory once for all layers of a step; with a plan a wave finds its unit's first tile (item, token, block
//     ids) in one record, fetched next to the copy, instead of a prefix sum, a search and a block-table fetch;
//   * a unit that crosses a sequence boundary emits one partial per sequence it touches, into slot
//     (unit index + sequence index), which is unique and contiguous per sequence; the merge kernel merges
//     the slots of each sequence and folds in the token being appended;
//   * block = 4 wave64; wave w owns KV head z*HW + w % HW, so with kv_heads >= 4 the four waves of a
//     workgroup read whole pages ([slot][kv_head][D] is contiguous).  Waves never synchronise after the
//     prologue.
// Data path per tile and wave (lane = (lr, lk) = (lane % 16, lane / 16); token group tg = 0 .. TK / 16 - 1):
//   K  global --16 B/lane--> registers --> MFMA A operand, no LDS: lane (lr, lk) fetches from token 16 tg + lr the
//      16-byte chunks lk, lk + 4, ... of the head's row, i.e. 64 contiguous bytes per token and load instruction.
//      The k index of the products is whatever dims those chunks hold; Q^T (B operand, in registers for the whole
//      sequence) is loaded in the same order, so S^T[token][head] = K . Q^T needs no shuffle.
//   V  global --same lane / chunk assignment--> registers --ds_write_b128--> LDS, chunk-major
//      ([token group][chunk][16 tokens][16 B]; 256 contiguous bytes per 16 lanes) --ds_read_b64_tr_b8 / _tr_b16-->
//      A operand V^T (the LDS transpose read gives each lane 8 tokens of one dim).  So that the 32 lanes of one pass of
//      the transpose read cover all 64 banks once, every odd token group starts 128 bytes off a multiple of 256 and,
//      for 16-bit elements (one read touches an even and an odd chunk), an odd chunk keeps its token rows 8..15 in
//      front of rows 0..7.
//   online softmax in the log2 domain on the C layout of S^T (head = lane % 16, 4 tokens per lane and group), once
//      per tile; the per-token K scale multiplies S, the V scale multiplies P (scales travel through LDS).
//   O^T[dim][head] += V^T . P^T per pair of token groups, where P^T *is* the C layout of S^T, so no cross-lane
//      movement of P is needed.
// One tile is in flight per wave: the loads of tile x + 1 go out while tile x is computed (V registers are free once
// the tile is staged, K registers once the scores are issued), the block ids of tile x + 2 in front of them.  (Moving
// the K tile to registers of its own so that its successor's loads go out at the start of the step was measured and
// changed nothing: the memory system, not the moment of issue, sets a tile's time.)  The
// loop over the tiles of a segment has no branches around loads, so every wait the compiler places counts
// exactly the loads younger than the one needed.
// int8 codes become fp16 by placing (code ^ 0x80) under the exponent byte 0x64 (v_perm): 1152 + code exactly;
// the offsets are removed algebraically (1152 * sum(q) per head, 1152 * sum(p) per head).  fp8 uses
// v_cvt_scalef32_pk_f16_fp8 with scale 1 (exact).  bf16 / fp16 caches feed the MFMA directly.
//
// The single-token append (areno/accel/csrc/attention.cu:526-553) is not part of this kernel: the streaming waves
// read the tokens that are in the pages, and the merge launch, which owns each (row, head) anyway, quantizes the
// new row, stores it and folds it in as one more partial (paged_decode.hip).
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
// tokens per tile step: a wave keeps one tile (K and V) in flight, 8 KB (8-bit) / 16 KB (16-bit) at head dim 128
#ifndef ARENO_MFMA_QUANT_TK
#define ARENO_MFMA_QUANT_TK 32
#endif
#ifndef ARENO_MFMA_WIDE_TK
#define ARENO_MFMA_WIDE_TK 32
#endif

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(2))) int int2_t;
typedef __attribute__((ext_vector_type(4))) int int4_t;

// Tokens per tile step of the kernel that serves a cache kind.
constexpr int decode_tile_tokens(bool quantized) { return quantized ? ARENO_MFMA_QUANT_TK : ARENO_MFMA_WIDE_TK; }

// What a plan (areno_hip_paged_decode_plan) holds for the split and merge kernels, all int32 in device memory:
//   cum    [items + 1]   exclusive prefix sums of the items' extents on the cost line (decode_items.hpp)
//   items  [items][4]    lo, end, row, nseq of every item
//   units  [units][16]   where a wave's unit starts (layout below)
//   rows   [batch][4]    for the merge kernel: first unit and number of units of the row's own item, and of its
//                        sub-group's shared item
constexpr int kDecodeDumpFloats = 16 * 512 + 2 * kWave;  // 16 columns of the widest head, and an (m, l) pair per lane
constexpr int kDecodeHold = 2;  // partials a wave parks in LDS before it stores them
constexpr int kPlanUnitWords = 16;
constexpr int kPlanUnitIds = 6;  // block ids of the first tile's columns that a unit record can hold
enum PlanUnitWord {
  kPuItem = 0,
  kPuTok = 1,
  kPuSegEnd = 2,
  kPuQEnd = 3,
  kPuQ0 = 4,  // the unit's positions on the cost line; q0 == q1: it holds no quantum
  kPuQ1 = 5,
  kPuLo = 6,
  kPuEnd = 7,
  kPuRow = 8,
  kPuNseq = 9,
  kPuIds = 10  // .. 15: block ids of columns (tok >> bs_shift) + 0 .. 5 of the item's row (clamped)
};

struct MfmaDecodeParams {
  DecodeParams d;      // part_ml / part_acc are indexed [slot][q_head] here
  int32_t* cum_out;    // [items + 1]: the prefix sums, written by workgroup 0 for the merge kernel (launches without a plan)
  int32_t tok_splits;  // waves of a workgroup that share a KV head (waves per workgroup / heads_per_wg / head split)
  int32_t num_units;   // gridDim.x * tok_splits
  int32_t head_parts;  // column tiles per kv head: ceil(q heads per kv head / 16); a wave serves one (kv head, part)
  // token -> block-table column for any page size: (token * bs_magic) >> (32 + bs_post), exact for tokens below 2^30
  // (page_division() in paged_decode.hip)
  uint32_t bs_magic;
  int32_t bs_post;
  ItemShape items;     // rows -> items (prefix groups, window, whether the merge folds in the token being appended)
  // A plan built once for all layers of a step (NULL: every workgroup derives the work list from the lengths).
  const int32_t* plan_cum;
  const int32_t* plan_items;
  const int32_t* plan_units;
  const int32_t* plan_rows;
  // The token being appended, for the merge kernel when items.append_in_merge: [batch, kv_heads, head_dim], dtype
  // q_dtype; quantized like the cache writer does and stored into the page.
  const void* k_update;
  const void* v_update;
  int32_t write_append;  // 1: the merge stores the row into its page; 0: it only folds it in (the page holds it already)
  int64_t num_blocks;    // pages of the pool (the append skips a row whose page id lies outside)
  // Prefix groups (GROUPED kernels only): rows [i * group_rows, (i + 1) * group_rows) share the pages of their first
  // shared_lens[i] tokens.  Shared items leave their partials in a second region (16 columns per kv head and slot).
  const int32_t* shared_lens;  // [batch / group_rows]
  float* shared_ml;            // [slot][kv_head][16][2]
  float* shared_acc;           // [slot][kv_head][16][head_dim]
  float* dump;                 // kDecodeDumpFloats floats that the lanes without a partial row store to; never read
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

// maximum of N values in ceil((N - 1) / 2) instructions (v_max3_f32)
template <int N>
__device__ __forceinline__ float max_all(const float (&v)[N]) {
  if constexpr (N == 1) {
    return v[0];
  } else if constexpr (N == 2) {
    return max_f32(v[0], v[1]);
  } else {
    constexpr int M = (N + 2) / 3;
    float r[M];
#pragma unroll
    for (int i = 0; i < N / 3; ++i) r[i] = max3_f32(v[3 * i], v[3 * i + 1], v[3 * i + 2]);
    if constexpr (N % 3 == 2) r[M - 1] = max_f32(v[N - 2], v[N - 1]);
    if constexpr (N % 3 == 1) r[M - 1] = v[N - 1];
    return max_all<M>(r);
  }
}

// a wave-uniform value that the compiler cannot prove uniform (it came out of LDS): move it to a scalar register
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

// The item table in LDS as the cursor functions of decode_items.hpp want it; the lookups' indices are the same in
// all lanes of a wave, so the values end up in scalar registers.
struct LdsItemTable {
  const int4_t* item;  // lo, end, row, nseq
  const int* cum_;
  __device__ __forceinline__ ItemInfo info(int b) const {
    const int4_t r = item[b];
    ItemInfo it;
    it.lo = uniform(r[0]);
    it.end = uniform(r[1]);
    it.row = uniform(r[2]);
    it.nseq = uniform(r[3]);
    return it;
  }
  __device__ __forceinline__ int cum(int i) const { return uniform(cum_[i]); }
};

// The sequence lengths in LDS (grouped launches) or in device memory, for item_info in the prologue.
struct LdsLens {
  const int* len;
  const int* glen;
  __device__ __forceinline__ int row_len(int b) const { return len[b]; }
  __device__ __forceinline__ int group_len(int g) const { return glen[g]; }
};

// What the pipeline remembers of a tile between the moment its block ids are requested and the moment it is computed
// (all wave-uniform).
struct TileDesc {
  int tok;    // first token of the tile inside its sequence
  int end;    // end of the segment the tile belongs to (tokens at and behind it are masked)
  int row;    // block-table / query row
  int nseq;   // rows side by side (shared items), else 1
  int b;      // item index
  int q_end;  // where the segment ends on the cost line
  int kind;   // kTilePhantom: past the unit's end
};
constexpr int kTilePhantom = 4;

// DSPLIT > 1 serves heads of DSPLIT * D elements (256 = 2 x 128, 192 = 3 x 64, 512 = 4 x 128): DSPLIT adjacent waves
// of the workgroup take one part of the head dimension each.  Every wave computes the part of S = K . Q^T over its
// elements, the waves exchange the parts through LDS, add them in the same order and go on with identical scores:
// the same softmax in all, P . V over the wave's own part of V, the wave's part of the partial row.  The waves of a
// head synchronise through two counters each in LDS (part ready / parts consumed); no workgroup barrier is involved,
// so the heads of one workgroup may run different units.
// The arguments in front of the parameter block are what a wave's first loads are addressed with (its unit's record
// and the plan's tables, or the sequence lengths): as leading scalar arguments they reach the wave in registers at its
// start (kernel-argument preload; the build asks for up to 16 words), so the first fetch does not wait for a fetch of
// the argument block -- one dependent memory round trip less at the start of every launch (0.5 us of ~30).
template <int KIND, int D, bool SCALE16, int NW, bool GROUPED = false, int DSPLIT = 1,
          int TK = decode_tile_tokens(KVTraits<KIND>::kQuant)>
__global__ __launch_bounds__(NW * kWave, KVTraits<KIND>::kQuant ? ARENO_MFMA_QUANT_OCC : ARENO_MFMA_WIDE_OCC) void decode_mfma_kernel(
    const int32_t* plan_units, const int32_t* plan_items, const int32_t* plan_cum, const int32_t* cache_seqlens,
    int32_t tok_splits, int32_t heads_per_wg, int32_t num_items, MfmaDecodeParams mp) {
  using T = KVTraits<KIND>;
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using Pair = typename T::pair_t;
  const DecodeParams& p = mp.d;
  constexpr int ES = T::kBytes;
  constexpr int NTG = TK / 16;         // token groups of 16 per tile
  constexpr int NPP = NTG / 2;         // pairs of token groups: one P.V product per pair and dim block
  constexpr int CPT = D * ES / 16;     // 16-byte chunks per token row
  constexpr int CPL = CPT / 4;         // chunks per lane and token: lk, lk + 4, ...
  constexpr int NS = D / 32;           // QK^T k-slices
  constexpr int NB = D / 16;           // P.V dim blocks
  constexpr int WPS = 8 * ES / 4;      // dwords per k-slice of 8 elements
  constexpr int TGS = CPT * 256 + 128;    // bytes of one token group of the V tile in LDS (128 of padding behind it)
  constexpr int SPL = 2 * TK / kWave;  // scale entries (K scales of the tile's tokens, then V scales) per lane
  constexpr float kPScale = T::kQuant ? 256.0f : 1.0f;
  constexpr int kParkFloats = DSPLIT > 1 ? 4 * NTG * kWave : 0;
  constexpr int kWaveLds = NTG * TGS + 2 * TK * 4 + kParkFloats * 4;
  static_assert(CPL >= 1 && CPL <= 4 && (D == 64 || D == 128), "unsupported head_dim");
  static_assert(TK == 32 || TK == 64, "a tile is two or four groups of 16 tokens");
  static_assert(DSPLIT == 1 || (DSPLIT >= 2 && DSPLIT <= 4 && !GROUPED && NW % DSPLIT == 0), "unsupported head split");
  constexpr int DFULL = D * DSPLIT;  // elements of a whole head (row of Q, of a cache page, of a partial)

  __shared__ __attribute__((aligned(16))) char s_tiles[NW][kWaveLds];
  constexpr int kMaxItems = (GROUPED ? 2 : 1) * kMfmaMaxBatch;  // at most one shared item per row on top of the rows
  __shared__ __attribute__((aligned(16))) int4_t s_item[kMaxItems];
  __shared__ int s_cum[kMaxItems + 1];
  __shared__ int s_wave_tot[NW];
  __shared__ int s_len[GROUPED ? kMfmaMaxBatch : 1];            // sequence lengths of the rows
  constexpr int kMaxGroups = kMfmaMaxBatch / 2;                 // groups have at least two rows
  __shared__ int s_group_len[GROUPED ? kMaxGroups : 1];         // shared prefix length of each group
  __shared__ __attribute__((aligned(16))) float s_hold[NW][kDecodeHold][kWave * 4 * (NB + 1)];  // parked partials
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

  const ItemShape& shape = mp.items;
  const LdsItemTable table = {s_item, s_cum};
  const bool planned = plan_units != nullptr;  // (scalar)

  const int hw_count = heads_per_wg;
  const int half = wave % DSPLIT;  // which part of the head dimension this wave owns
  const int hw = (wave / DSPLIT) % hw_count;
  const int ts = (wave / DSPLIT) / hw_count;
  // more than 16 query heads per kv head take several column tiles: the "heads" the grid is laid out over are
  // (kv head, part) pairs, the parts of a kv head next to each other so that they stream its pages at the same time
  const int vhead = blockIdx.y * hw_count + hw;
  const int kvh = mp.head_parts > 1 ? vhead / mp.head_parts : vhead;
  const int part = vhead - kvh * mp.head_parts;
  const int group_here = min(16, p.group - 16 * part);  // query heads of this wave's column tile
  const int unit = blockIdx.x * tok_splits + ts;

  // ---- the item table: (lo, end, row, nseq) of every item and the exclusive prefix sum of their quanta, in LDS -----
  int q0 = 0, q1 = 0;       // this wave's unit
  TileCursor cur;           // the furthest tile requested so far
  int first_ids[kPlanUnitIds];  // with a plan: block ids of the first tile's columns
  if (planned) {
    // the wave's unit record (one 64-byte scalar fetch), and the workgroup's copy of the plan's tables
    const int32_t* rec = plan_units + static_cast<int64_t>(unit) * kPlanUnitWords;
    q0 = rec[kPuQ0];
    q1 = rec[kPuQ1];
    cur.b = rec[kPuItem];
    cur.tok = rec[kPuTok];
    cur.seg_end = rec[kPuSegEnd];
    cur.q_end = rec[kPuQEnd];
    cur.it.lo = rec[kPuLo];
    cur.it.end = rec[kPuEnd];
    cur.it.row = rec[kPuRow];
    cur.it.nseq = rec[kPuNseq];
#pragma unroll
    for (int i = 0; i < kPlanUnitIds; ++i) first_ids[i] = rec[kPuIds + i];
    for (int v = tid; v <= num_items; v += NW * kWave) {
      if (v < num_items) s_item[v] = *reinterpret_cast<const int4_t*>(plan_items + 4 * static_cast<int64_t>(v));
      s_cum[v] = plan_cum[v];
    }
    if (lane == 0) s_pair_flags[0][wave] = s_pair_flags[1][wave] = 0;
    __syncthreads();
  } else {
    int nt[SPT];
    int local = 0;
    if constexpr (GROUPED) {
      // an item's extent takes the group's length, its members' lengths and the row's own: the workgroup copies both
      // arrays with independent loads first (the launcher sends at most kMfmaMaxBatch rows in groups of >= 2)
      for (int i = tid; i < shape.batch; i += NW * kWave) s_len[i] = cache_seqlens[i];
      for (int i = tid; i < shape.num_groups(); i += NW * kWave) s_group_len[i] = mp.shared_lens[i];
      __syncthreads();
      const LdsLens lens = {s_len, s_group_len};
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        nt[j] = 0;
        if (v < num_items) {
          const ItemInfo it = item_info<true>(shape, lens, v);
          s_item[v] = int4_t{it.lo, it.end, it.row, it.nseq};
          nt[j] = it.extent(shape.switch_quanta);
        }
        local += nt[j];
      }
    } else {
      // the thread's sequence lengths are fetched together (clamped index, no branch around the load)
      int len[SPT];
#pragma unroll
      for (int j = 0; j < SPT; ++j) len[j] = cache_seqlens[min(SPT * tid + j, num_items - 1)];
#pragma unroll
      for (int j = 0; j < SPT; ++j) {
        const int v = SPT * tid + j;
        nt[j] = 0;
        if (v < num_items) {
          ItemInfo it;
          it.lo = first_visible_key(len[j] + 1, shape.window_left);
          it.end = len[j] + 1 - shape.append_in_merge;
          it.row = v;
          it.nseq = 1;
          s_item[v] = int4_t{it.lo, it.end, it.row, it.nseq};
          nt[j] = it.extent(shape.switch_quanta);
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
    const UnitGeometry geo = make_unit_geometry(table.cum(num_items), mp.num_units);
    if (blockIdx.x == 0 && blockIdx.y == 0) {
      for (int v = tid; v <= num_items; v += NW * kWave) mp.cum_out[v] = s_cum[v];
    }
    q0 = geo.unit_start(unit);
    q1 = geo.unit_start(unit + 1);
    if (q0 < q1 && !cursor_seek(cur, table, shape.switch_quanta, num_items, q0, q1)) q1 = q0;  // no quantum in the unit
  }
  ARENO_TRACE_POINT();

  char* const v_tile = &s_tiles[wave][0];
  float* const sc_lds = reinterpret_cast<float*>(&s_tiles[wave][NTG * TGS]);  // [0, TK): K scales, [TK, 2 TK): V scales
  float* const park = reinterpret_cast<float*>(&s_tiles[wave][NTG * TGS + 2 * TK * 4]);

  constexpr int64_t row_bytes = static_cast<int64_t>(DFULL) * ES;
  const int64_t half_bytes = static_cast<int64_t>(half) * D * ES;  // of this wave's part inside a cache / update row
  const int h0 = kvh * p.group + 16 * part;
  const bool q_is_operand_type = (KIND == KV_BF16 && p.q_dtype == ARENO_DT_BF16) ||
                                 (KIND != KV_BF16 && p.q_dtype == ARENO_DT_F16);
  auto is_shared = [&](int v) { return GROUPED && v < shape.num_shared; };
  // first element of the 8 that k-slice sl holds in this lane (the chunk order of the K loads)
  auto slice_base = [&](int sl) { return ES == 1 ? 16 * (lk + 4 * (sl >> 1)) + 8 * (sl & 1) : 8 * (lk + 4 * sl); };
  // byte offset of token row r (0..15) of chunk c inside a token group of the V tile: 16-bit tiles keep the two
  // halves of an odd chunk's rows swapped (see the layout note above)
  auto chunk_row_pos = [](int c, int r) { return c * 256 + ((ES == 2 && (c & 1)) ? (r ^ 8) : r) * 16; };
  // byte offset of token group tg inside the V tile: odd groups 128 bytes off a multiple of 256
  auto group_pos = [](int tg) { return tg * TGS; };

  // ---- the pipeline's registers ------------------------------------------------------------------------------------
  // Every step issues the same loads in the same order whatever the tiles involved (only their addresses differ), so
  // that the waits the compiler places count exactly the loads that are younger than the one needed and the tiles
  // behind it stay in flight.  The Q of the next item is an extra load at the start of a segment.
  typedef typename std::conditional<SCALE16, uint16_t, float>::type scale_raw_t;
  uint4_t kreg[NTG * CPL], vreg[NTG * CPL];
  scale_raw_t sreg[SPL];  // entry lane + 64 i of [K scales of the tile's tokens, V scales of the tile's tokens]
  TileDesc desc0;      // the tile whose loads are in the registers
  TileDesc desc_ids;   // the furthest tile requested so far (its block ids are on their way)

  auto describe = [&](const TileCursor& c) {
    TileDesc t;
    t.tok = c.tok;
    t.end = c.seg_end;
    t.row = c.it.row;
    t.nseq = c.it.nseq;
    t.b = c.b;
    t.q_end = c.q_end;
    t.kind = 0;
    return t;
  };
  // block-table column and slot of a token, for any page size: a division by multiply and shift
  auto column_of = [&](int t) { return static_cast<int>(__umulhi(static_cast<uint32_t>(t), mp.bs_magic) >> mp.bs_post); };
  auto slot_of = [&](int t) { return t - column_of(t) * p.block_size; };
  // The token whose cache row this lane fetches for group tg: its own token of the tile, clamped to the segment's
  // last one; one token for all lanes of a phantom tile (a tile past the unit's end: its loads keep the pipeline's
  // shape and hit one cache line each).
  auto lane_token = [&](const TileDesc& t, int tg) {
    const int own = (t.kind & kTilePhantom) ? 0 : 16 * tg + lr;
    return max(min(t.tok + own, t.end - 1), 0);  // (never negative: the page division below takes it as unsigned)
  };
  // (block ids and cache rows are indexed with compile-time constants only: an array indexed by a lane-dependent
  // value would live in scratch memory, and scratch loads count with the global loads and drain the pipeline)
  struct IdSet {
    int g[NTG];
  };
  auto issue_id_loads = [&](const TileDesc& t) {
    const int32_t* table_row = p.block_table + static_cast<int64_t>(t.row) * p.max_blocks;
    IdSet r;
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) r.g[tg] = table_row[column_of(lane_token(t, tg))];
    return r;
  };
  // cache row (block, slot, head) of this lane's token of each group, from the block ids that have arrived
  uint32_t row_g[NTG];
  auto rows_from_ids = [&](const TileDesc& t, const IdSet& src) {
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg)
      row_g[tg] = (static_cast<uint32_t>(src.g[tg]) * p.block_size + slot_of(lane_token(t, tg))) * p.kv_heads + kvh;
  };
  auto issue_v_loads = [&]() {
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
      const char* va = static_cast<const char*>(p.v_cache) + row_g[tg] * row_bytes + half_bytes + lk * 16;
#pragma unroll
      for (int j = 0; j < CPL; ++j) vreg[tg * CPL + j] = *reinterpret_cast<const uint4_t*>(va + 64 * j);
    }
    if constexpr (T::kQuant) {
      // entry e = lane + 64 i is the scale of token e % TK = 16 (lk % NTG) + lr, whose cache row this lane holds
      uint32_t r = row_g[0];
#pragma unroll
      for (int tg = 1; tg < NTG; ++tg) r = (lk % NTG) == tg ? row_g[tg] : r;
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const bool is_v = (lane + kWave * i) >= TK;
        sreg[i] = static_cast<const scale_raw_t*>(is_v ? p.v_scale : p.k_scale)[r];
      }
    }
  };
  auto issue_k_loads = [&]() {
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
      const char* ka = static_cast<const char*>(p.k_cache) + row_g[tg] * row_bytes + half_bytes + lk * 16;
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
  // slice for 16-bit queries.  Column lr of the MFMA tiles: head lr of the row in a per-row item, (row lr / G, head
  // lr % G) in a shared item.  The first step of a segment fetches the Q of the item that follows the segment; the
  // next item adopts it when the segment is done.  (A column without a head fetches the row of the item's first head,
  // which adopt_q drops.)
  uint4_t qraw[NS];
  bool q_live = false;          // whether this lane's column has a head in the item q_src points into
  const char* q_src = nullptr;  // this lane's part of the Q row that the steps fetch
  const int col_seq = GROUPED ? lr / p.group : 0;
  const int col_head = GROUPED ? lr - col_seq * p.group : lr;
  auto set_q_source = [&](int item, int row, int nseq) {
    const bool shared = is_shared(item);
    const int m = shared ? col_seq : 0;
    const int g = shared ? col_head : lr;
    const bool live = shared ? m < nseq : lr < group_here;
    const int64_t head_row = live ? static_cast<int64_t>(row + m) * p.q_heads + h0 + g
                                  : static_cast<int64_t>(row) * p.q_heads + h0;
    q_live = live;
    q_src = static_cast<const char*>(p.q) + (head_row * DFULL + half * D) * 2;
  };
  auto issue_q_loads = [&]() {
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) qraw[sl] = load16(q_src, slice_base(sl) * 2);
  };
  V8 qop[NS];
  float qbias = 0.0f;
  float4_t score_init = {0.0f, 0.0f, 0.0f, 0.0f};  // what the score products accumulate onto: -qbias for int8, else 0
  auto adopt_q = [&]() {
    float qsum = 0.0f;
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      uint4_t w = qraw[sl];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = q_live ? w[j] : 0u;
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
  // taken out with; from the matrix cores (an all-ones A operand puts the column's sum over a pair's 32 tokens, all
  // four k groups included, into every element), like the products it corrects
  float4_t p_sum = {0.0f, 0.0f, 0.0f, 0.0f};
  auto reset_state = [&]() {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    m_run = kNegInf;
    l_run = 0.0f;
    p_sum = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  };

  auto lds_fence = [&]() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // A finished segment's partial: the un-normalised accumulator rows and (m, l) of every column.  Per-row items go to
  // slot unit + row, one row per q head; shared items to slot unit + item, 16 columns per kv head.  Every lane stores
  // (no branch): columns without a head, and the (m, l) pair of the lanes that do not own it, go to a dump row that
  // nothing reads.
  auto store_partial = [&](int v, int row, int nseq, const float4_t (&o)[NB], float m_val, float l_val) {
    const bool shared = is_shared(v);
    const bool live = shared ? col_seq < nseq : lr < group_here;
    const int64_t prow = shared ? (static_cast<int64_t>(unit + v) * p.kv_heads + kvh) * 16 + lr
                                : static_cast<int64_t>(unit + row) * p.q_heads + h0 + lr;
    float* const ml = shared ? mp.shared_ml : p.part_ml;
    float* const rows = shared ? mp.shared_acc : p.part_acc;
    float* dst = (live ? rows + prow * DFULL : mp.dump + lr * DFULL) + half * D + 4 * lk;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) *reinterpret_cast<float4_t*>(dst + 16 * nb) = o[nb];
    float* const ml_dst = (live && lk == 0) ? ml + prow * 2 : mp.dump + 16 * DFULL + 2 * lane;
    *reinterpret_cast<float2_t*>(ml_dst) = float2_t{m_val, l_val};
  };
  auto partial_values = [&](float4_t (&o)[NB], float& l_tot) {
    // combine the four k-groups' row sums; every lane of a head ends with the head's totals
    l_tot = rows_sum(l_run);
    float off = 0.0f;
    if constexpr (KIND == KV_I8) off = kI8Offset * p_sum[0];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) o[nb][j] = (acc[nb][j] - off) * (1.0f / kPScale);
    }
  };
  // The partial of a segment behind which the unit goes on is parked in LDS and stored when the unit is done.  A
  // store in the middle of the tile stream would sit in front of every later load in the wave's memory queue, which
  // retires in order: each wait for a tile behind it would also wait for the stores' acknowledgement (measured: 2.4 us
  // of a 32.7 us launch on units with two segments).  kDecodeHold partials fit; a unit with more segments stores the
  // parked ones when the space is full.
  int held = 0;
  auto hold_slot = [&](int k) { return reinterpret_cast<float4_t*>(&s_hold[wave][k][0]) + lane; };
  auto park_partial = [&](int v, int row, int nseq) {
    float4_t o[NB];
    float l_tot;
    partial_values(o, l_tot);
    float4_t* slot = hold_slot(held);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) slot[nb * kWave] = o[nb];
    slot[NB * kWave] = float4_t{m_run, l_tot, __builtin_bit_cast(float, v), __builtin_bit_cast(float, (row << 5) | nseq)};
    ++held;
  };
  auto flush_parked = [&]() {
    lds_fence();
    for (int k = 0; k < held; ++k) {
      const float4_t* slot = hold_slot(k);
      float4_t o[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) o[nb] = slot[nb * kWave];
      const float4_t tail = slot[NB * kWave];
      // (copies first: a bit_cast straight from a vector-element lvalue reads element 0)
      const float item_bits = tail[2], rows_bits = tail[3];
      const int v = uniform(__builtin_bit_cast(int, item_bits));
      const int rn = uniform(__builtin_bit_cast(int, rows_bits));
      store_partial(v, rn >> 5, rn & 31, o, tail[0], tail[1]);
    }
    held = 0;
  };
  auto write_partial = [&](int v, int row, int nseq) {
    float4_t o[NB];
    float l_tot;
    partial_values(o, l_tot);
    store_partial(v, row, nseq, o, m_run, l_tot);
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

  // ---- one tile: stage V and the scales, scores, softmax, P.V ------------------------------------------------------
  // `between_v` runs once the V registers are free, `between_k` once the K registers are.
  auto tile_step = [&](const TileDesc& t, auto&& between_v, auto&& between_k) {
    if constexpr (DSPLIT > 1) {
      // the other waves of the head must have read the score part this wave parked in the previous step
#pragma unroll
      for (int part = 0; part < DSPLIT; ++part) {
        if (part != half) pair_wait(&s_pair_flags[1][wave - half + part], pair_step);
      }
    }
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        uint4_t vv = vreg[tg * CPL + j];
        if constexpr (KIND == KV_I8) {
#pragma unroll
          for (int w = 0; w < 4; ++w) vv[w] ^= kI8Flip;
        }
        *reinterpret_cast<uint4_t*>(v_tile + group_pos(tg) + chunk_row_pos(lk + 4 * j, lr)) = vv;
      }
    }
    if constexpr (T::kQuant) {
#pragma unroll
      for (int i = 0; i < SPL; ++i) {
        const int e = lane + kWave * i;
        const bool is_v = e >= TK;
        const bool ok = t.tok + (e & (TK - 1)) < t.end;
        const float s = scale_value(sreg[i]);
        sc_lds[e] = is_v ? (ok ? s * kPScale : 0.0f) : (ok ? s * p.scale_log2e : kNegInf);
      }
    }
    lds_fence();
    between_v();  // the V registers are free

    // -- S^T = K . Q^T for the 16-token groups ----------------------------------------------------------------------
    float s[NTG][4];
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
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
      // dimension.  Every wave of the head ends up with the same sums.
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
        for (int j = 0; j < 4; ++j) park[(4 * tg + j) * kWave + lane] = s[tg][j];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      ++pair_step;
      if (lane == 0)
        __hip_atomic_store(&s_pair_flags[0][wave], pair_step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      const int first_wave = wave - half;
      float total[NTG][4];
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
        for (int j = 0; j < 4; ++j) total[tg][j] = 0.0f;
      }
#pragma unroll
      for (int part = 0; part < DSPLIT; ++part) {
        if (part == half) {
#pragma unroll
          for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) total[tg][j] += s[tg][j];
          }
        } else {
          pair_wait(&s_pair_flags[0][first_wave + part], pair_step);
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
          const float* theirs = reinterpret_cast<const float*>(&s_tiles[first_wave + part][NTG * TGS + 2 * TK * 4]);
#pragma unroll
          for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) total[tg][j] += theirs[(4 * tg + j) * kWave + lane];
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // the reads above are done before the others hear
      if (lane == 0)
        __hip_atomic_store(&s_pair_flags[1][wave], pair_step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
        for (int j = 0; j < 4; ++j) s[tg][j] = total[tg][j];
      }
    }
    // the per-token K scale (softmax scale and log2 e folded in); tokens past the end become exactly -inf, which only
    // a segment's last tile has: every other tile takes the branch with one multiply per score
    float vs[NTG][4];
    const bool whole_tile = t.tok + TK <= t.end;  // (scalar)
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
      if constexpr (T::kQuant) {
        const float4_t vv = *reinterpret_cast<const float4_t*>(sc_lds + TK + 16 * tg + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) vs[tg][j] = vv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) vs[tg][j] = 1.0f;
      }
    }
    if (whole_tile) {
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
        float4_t ks = {p.scale_log2e, p.scale_log2e, p.scale_log2e, p.scale_log2e};
        if constexpr (T::kQuant) ks = *reinterpret_cast<const float4_t*>(sc_lds + 16 * tg + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) s[tg][j] *= ks[j];
      }
    } else {
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
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

    // -- online softmax for column lr over the tile's tokens ---------------------------------------------------------
    float flat[4 * NTG];
#pragma unroll
    for (int tg = 0; tg < NTG; ++tg) {
#pragma unroll
      for (int j = 0; j < 4; ++j) flat[4 * tg + j] = s[tg][j];
    }
    const float mt = rows_max(max_all<4 * NTG>(flat));
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
    V8 pop[NPP];
#pragma unroll
    for (int pp = 0; pp < NPP; ++pp) {
      float pe[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e0 = fast_exp2(s[2 * pp][j] - m_safe);
        const float e1 = fast_exp2(s[2 * pp + 1][j] - m_safe);
        l_run += e0 + e1;
        pe[j] = T::kQuant ? e0 * vs[2 * pp][j] : e0;
        pe[4 + j] = T::kQuant ? e1 * vs[2 * pp + 1][j] : e1;
      }
      uint32_t pw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) pw[j] = pack_pair<KIND>(pe[2 * j], pe[2 * j + 1]);
      pop[pp] = __builtin_bit_cast(V8, uint4_t{pw[0], pw[1], pw[2], pw[3]});
      if constexpr (KIND == KV_I8) {
        constexpr uint32_t kOnes = 0x3c003c00u;  // two fp16 1.0
        p_sum = Ops::mfma(__builtin_bit_cast(V8, uint4_t{kOnes, kOnes, kOnes, kOnes}), pop[pp], p_sum);
      }
    }

    // -- O^T += V^T . P^T, one MFMA per 16-dim block and pair of token groups ----------------------------------------
#pragma unroll
    for (int pp = 0; pp < NPP; ++pp) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        uint32_t vw[4];
        if constexpr (ES == 1) {
          // lane i of a 16-lane group supplies token row (i / 2), 8 bytes at column 8 (i % 2) of chunk nb: rows 0..3 are
          // tokens 4 lk .. 4 lk + 3 of the pair's first group, rows 4..7 the same tokens of its second group
          const int r8 = lr >> 1;
          const int tg = 2 * pp + (r8 >> 2);
          const int tok = 4 * lk + (r8 & 3);
          char* a = v_tile + group_pos(tg) + chunk_row_pos(nb, tok) + 8 * (lr & 1);
          const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_int2*)a);
          vw[0] = static_cast<uint32_t>(r[0]);
          vw[1] = static_cast<uint32_t>(r[1]);
        } else {
          // lane i supplies token row (i / 4), 4 elements at column 4 (i % 4) of the 16-dim block: chunk 2 nb + (i % 4) / 2,
          // byte 8 ((i % 4) % 2); two reads of 4 tokens, one per token group
          const int r4 = lr >> 2;
          const int c4 = lr & 3;
#pragma unroll
          for (int g2 = 0; g2 < 2; ++g2) {
            char* a = v_tile + group_pos(2 * pp + g2) + chunk_row_pos(2 * nb + (c4 >> 1), 4 * lk + r4) + 8 * (c4 & 1);
            const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
            const uint2_t u = __builtin_bit_cast(uint2_t, r);
            vw[2 * g2] = u[0];
            vw[2 * g2 + 1] = u[1];
          }
        }
        acc[nb] = Ops::mfma(to_operand<KIND>(vw), pop[pp], acc[nb]);
      }
    }
    // all LDS reads of this tile are done before the next step overwrites it
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- this wave's unit --------------------------------------------------------------------------------------------
  if (q0 < q1) {
    // move the request cursor one tile on (to a phantom past the unit's end) and ask for that tile's block ids
    IdSet ids;  // block ids of the tile the request cursor is on
    auto request_next = [&]() {
      if (!(desc_ids.kind & kTilePhantom)) {
        const CursorMove mv = cursor_advance(cur, table, shape.switch_quanta, q1, TK);
        if (mv == kCursorUnitDone) {
          desc_ids.kind = kTilePhantom;
        } else {
          desc_ids = describe(cur);
        }
      }
      ids = issue_id_loads(desc_ids);
    };
    // ---- prologue: block ids of the first tile (from the unit record when there is a plan), Q of the first item,
    // the first tile's loads, block ids of the second tile ------------------------------------------------------------
    desc_ids = describe(cur);
    desc0 = desc_ids;
    IdSet ids_first;
    // a record's ids cover kPlanUnitIds columns from the first token's: enough unless pages are very small
    const bool ids_from_plan = planned && column_of(desc0.tok + TK - 1) - column_of(desc0.tok) < kPlanUnitIds;
    if (ids_from_plan) {
      const int col0 = column_of(desc0.tok);
#pragma unroll
      for (int tg = 0; tg < NTG; ++tg) {
        const int c = column_of(lane_token(desc0, tg)) - col0;
        int id = first_ids[0];
#pragma unroll
        for (int i = 1; i < kPlanUnitIds; ++i) id = c == i ? first_ids[i] : id;
        ids_first.g[tg] = id;
      }
    } else {
      ids_first = issue_id_loads(desc0);
    }
    set_q_source(desc0.b, desc0.row, desc0.nseq);
    issue_q_loads();
    request_next();  // the second tile's ids right behind the first tile's
    rows_from_ids(desc0, ids_first);
    issue_v_loads();
    issue_k_loads();
    adopt_q();
    reset_state();

    // One step of the pipeline on the tile in the registers (tile x): the ids of tile x + 1 have arrived (requested a
    // step ago), those of tile x + 2 are requested, and tile x + 1's loads go out as the step frees the V registers
    // (`between_v`) and the K registers (`between_k`).
    auto step = [&](auto first_of_segment) {
      ARENO_TRACE_POINT();
      const TileDesc t = desc0;
      const TileDesc nt = desc_ids;
      rows_from_ids(nt, ids);
      // the ids are consumed before the next ones are requested into the same registers
      __builtin_amdgcn_sched_barrier(0);
      request_next();
      if constexpr (decltype(first_of_segment)::value) issue_q_loads();
      // (scheduling barriers: a load of the next tile must not move in front of the last use of the registers it
      // fills, or the two values would need different registers and a copy of a value still in flight)
      tile_step(
          t,
          [&]() {
            __builtin_amdgcn_sched_barrier(0);
            issue_v_loads();
            __builtin_amdgcn_sched_barrier(0);
          },
          [&]() {
            __builtin_amdgcn_sched_barrier(0);
            issue_k_loads();
            __builtin_amdgcn_sched_barrier(0);
          });
      desc0 = nt;
    };

    // The unit as a sequence of segments: the tiles of one item that fall into the unit.  The loop over a segment's
    // tiles has no item logic in it (so nothing but the tile stream is carried around it); the partial and the switch
    // to the next item's Q come behind it.
    for (;;) {
      const TileDesc first = desc0;
      const int steps = (first.end - first.tok + TK - 1) / TK;
      // the next item the unit holds quanta of, if any: its Q is what this segment's first step fetches
      const int b2 = next_item_in_unit(table, shape.switch_quanta, first.b, first.q_end, q1);
      const bool more = b2 >= 0;
      if (more) {
        const ItemInfo it2 = table.info(b2);
        set_q_source(b2, it2.row, it2.nseq);
      }
      // The first step of a segment is a copy of its own that fetches the Q of the item that follows the segment (of
      // the segment's own item when none follows) at a fixed place in its load sequence, so no load sits behind a
      // branch and the waits the compiler places in either copy count exactly the loads that are in flight.
      step(std::true_type{});
      for (int i = 1; i < steps; ++i) step(std::false_type{});
      // the next item's Q first (its loads are older than a tile's), the partial's stores behind it
      if (!more) {
        write_partial(first.b, first.row, first.nseq);
        flush_parked();
        break;
      }
      adopt_q();
      if (held == kDecodeHold) flush_parked();
      park_partial(first.b, first.row, first.nseq);
      reset_state();
    }
  }
#ifdef ARENO_TRACE
  if (mp.trace && lane == 0) mp.trace[trace_wave * 8 + 6] = wall_clock64();
#endif
}

typedef void (*decode_mfma_fn)(const int32_t*, const int32_t*, const int32_t*, const int32_t*, int32_t, int32_t, int32_t,
                               MfmaDecodeParams);
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
