// Causal varlen prefill over paged (optionally quantized) KV on the matrix cores (gfx950).
//
// Work item = (sequence, kv head, block of query tokens).  The G query heads of the kv head are folded into the
// query-row axis: row r of the block is (token r / G, head r % G), so a block of 256 rows holds 256 / G tokens of
// all heads (36 of them for 7 heads: 4 rows stay empty, where padding G to 8 left 32) and K/V are read once for the
// whole group (GQA without expanding KV, as areno/accel/csrc/attention.cu:170-171 does per row; a kv head with more
// than 16 q heads runs as several workgroup rows, 16 q heads each).  A block is 256 rows: each of the 8 waves
// owns 32 (two 16-row tiles; one at head dims 192 and 256, and at 512 two waves share one).  One such workgroup per
// CU (the registers allow two waves per SIMD either way; eight waves behind one set of K/V tiles halve the staging
// work per wave against two workgroups of four).
//
// Balance: an item costs one "tile step" per 32-key tile it may see, and items differ by orders of magnitude (a
// query block on a 16k context next to one on an empty context).  Every workgroup computes the prefix sum of tile
// steps over the sequences in LDS and takes an equal share of the global tile-step range of its kv head (a "unit"),
// whatever the length distribution.  A unit is a run of segments, each a range of key tiles of one item:
//   * an item that lies inside one unit is finished there and written to `out`;
//   * an item cut by a unit border leaves un-normalised partials (running max, sum, accumulator) in the workspace
//     -- slot 2u for the first item of unit u, slot 2u + 1 for its last -- and prefill_merge_kernel combines them.
//
// One segment, per 32-key tile t (all waves share the K/V tiles in LDS):
//   * the threads fetch K four tiles and V three tiles ahead with 16-byte coalesced loads (block ids two more
//     tiles ahead; two register sets alternate, so a fetch has two tile steps to arrive) and publish them into
//     double-buffered LDS tiles one iteration before their first use, so one barrier per tile is enough (padded
//     rows, conflict free).  8-bit codes are dequantized (times the per-token
//     scale) by the thread that stages them, once per workgroup: the tiles in LDS are always 16-bit.  When a tile
//     has at most one chunk per thread (8-bit tiles, 16-bit tiles at head dim 64) the first four waves stage K and
//     the last four V, one chunk each;
//   * S^T[key][row] = K . Q^T of tile t + 1 is issued in the same basic block as the row maxima of tile t, so the
//     matrix cores have independent work while the vector ALU runs the softmax: A = K rows from LDS, B = Q^T in
//     registers; C has row = lane % 16, 4 keys per lane;
//   * causal / window mask only on tiles that cross a mask edge, online softmax in the log2 domain with the softmax
//     scale folded into the exponent's multiply-add.  The value the exponentials are taken against is raised (and
//     the accumulators rescaled) only when a tile exceeds it by more than 2^8: each lane checks its own scores and a
//     ballot decides for the wave, so most tiles skip the cross-lane maxima (v_permlane swaps over the four lanes
//     of a row) and the rescale;
//   * O^T[dim][row] += V^T . P^T : A = V^T through the LDS transpose reads, B = P^T (= the C layout of S^T); one
//     more product with an all-ones A operand accumulates the row sums of P.
// The tile loop is unrolled by two with the roles of the two score arrays swapped, so the scores of tile t + 1 are
// computed where the next step reads them (and the fetch register sets alternate with them).  Matrix-core, vector-ALU
// and LDS time add up more than they overlap here: per pair of tile steps on a SIMD (two waves) the 68 products keep
// the matrix core busy for 1 088 cycles and the vector ALU from issuing for about half of that, the ~104 plain
// vector instructions and 16 v_exp_f32 (~9 cycles) of each wave take ~1 230, and the CU's LDS, at one instruction
// per ~6 cycles whatever its width, ~1 050 for the 26 reads and stores per wave; the pair takes ~2 600.
// The LDS layouts are the 16-bit ones of the decode kernel (decode_mfma_kernels.hpp).  Semantics:
// _reference_attention with query_start = context_lens[s] (areno/accel/attention.py:25-41 in the reference); with
// context 0 it is the reference's varlen kernel (areno/accel/csrc/attention.cu:145-242).

#include "decode_mfma_kernels.hpp"
#include "prefill_steps.hpp"

namespace areno {

// LDS row that holds tile token t of the V tile: the second half is rotated by 4 rows so that the 8 tokens a
// lane group reads through the transpose load ({4g..4g+3} and {16+4g..16+4g+3}) sit in rows distinct mod 16.
// Workgroup barrier that orders LDS accesses only.  The waves of this kernel exchange data through LDS alone, and a
// barrier that also orders global memory waits for the acknowledgement of every output row stored before it (~3 us
// behind an item's end), together with every fetch in front of those stores.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ int v_row_of(int t) { return t < 16 ? t : 16 + ((t + 4) & 15); }

size_t prefill_mfma_workspace_bytes(int32_t kv_heads, int32_t head_dim);
int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* workspace, size_t workspace_bytes, void* stream);

namespace {

#ifndef ARENO_PREFILL_WAVES
#define ARENO_PREFILL_WAVES 8
#endif
constexpr int kPrefillWaves = ARENO_PREFILL_WAVES;
constexpr int kPrefillThreads = 64 * kPrefillWaves;
constexpr int kMaxRowTiles = 2;                                   // 16-row MFMA tiles per wave
constexpr int kMaxRowsPerWg = 16 * kMaxRowTiles * kPrefillWaves;
constexpr int kMaxPrefillSeqs = 1024;
constexpr int kPrefillTargetWgs = 2048 / kPrefillWaves;  // eight resident waves on each of the 256 CUs
constexpr int kMaxPrefillUnits = 512;   // per kv head

struct PrefillParams {
  const void* q;
  void* out;
  const void* k_cache;
  const void* v_cache;
  const void* k_scale;
  const void* v_scale;
  const int32_t* block_table;
  const int32_t* cu_seqlens_q;
  const int32_t* context_lens;
  float* part_ml;   // [2 * units][kv_heads * head_parts][rows_per_wg][2]
  float* part_acc;  // [2 * units][kv_heads * head_parts][rows_per_wg][head_dim]
  int32_t num_seqs;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t head_dim;
  int32_t group;        // q heads per kv head
  int32_t head_parts;   // workgroup rows (blockIdx.y) per kv head: ceil(group / 16); each takes up to 16 of its q heads
  // Row folding: row r of a query block is (token r / fold, q head r % fold of the part), fold = the q heads per kv
  // head (16 when a kv head runs as several parts).  The quotient comes from a multiplication: r < 512, fold <= 16.
  int32_t fold;
  int32_t fold_magic;    // ceil(2^16 / fold): r / fold == (r * fold_magic) >> 16 for r < 2^12
  int32_t block_tokens;  // rows_per_wg / fold: query tokens per item (the last rows of a block stay empty when fold
                         // does not divide rows_per_wg)
  int32_t block_size;
  int32_t bs_shift;   // log2 of the page size, or -1: then a key's column is __umulhi(key, bs_magic) >> bs_post
  uint32_t bs_magic;
  int32_t bs_post;
  int32_t max_blocks;
  int32_t window_left;
  int32_t q_dtype;
  int32_t units;        // per (kv head, part)
  int32_t rows_per_wg;  // query rows of one item: 64 per 16-row tile a wave owns
  float scale_log2e;
};

// Exclusive prefix sum of tile steps per sequence into s_cum[0 .. num_seqs] (all threads take part).
__device__ __forceinline__ void prefix_tile_steps(const PrefillParams& p, int tq, int* s_cum, int* s_wave_tot) {
  constexpr int SPT = kMaxPrefillSeqs / kPrefillThreads;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  int steps[SPT];
  int local = 0;
#pragma unroll
  for (int i = 0; i < SPT; ++i) {
    const int s = SPT * tid + i;
    steps[i] = 0;
    if (s < p.num_seqs) {
      const int n_new = p.cu_seqlens_q[s + 1] - p.cu_seqlens_q[s];
      const int ctx = p.context_lens != nullptr ? p.context_lens[s] : 0;
      steps[i] = sequence_steps(n_new, ctx, tq, p.window_left);
    }
    local += steps[i];
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
  for (int i = 0; i < SPT; ++i) {
    const int s = SPT * tid + i;
    if (s <= p.num_seqs) s_cum[s] = excl;
    excl += steps[i];
  }
  // the entry behind the last thread's sequences has no owner of its own: it is the total when the list is full
  if (tid == kPrefillThreads - 1 && SPT * (tid + 1) <= p.num_seqs) s_cum[SPT * (tid + 1)] = excl;
  __syncthreads();
}

// Where global tile step x lies: sequence, query block, key tile.
struct StepPos {
  int seq, j, tile;
  int n_new, ctx;
  int q_begin;  // row of the sequence's first new token in q / out (cu_seqlens_q[seq])
  int item_x0;  // global step of the item's first tile
};

__device__ __forceinline__ StepPos locate_step(const PrefillParams& p, const int* s_cum, int tq, int x) {
  StepPos r;
  int lo = 0, hi = p.num_seqs;
  while (lo + 1 < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_cum[mid] <= x) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  r.seq = lo;
  r.q_begin = p.cu_seqlens_q[lo];
  r.n_new = p.cu_seqlens_q[lo + 1] - r.q_begin;
  r.ctx = p.context_lens != nullptr ? p.context_lens[lo] : 0;
  const int off = x - s_cum[lo];
  if (r.n_new <= 0 || off < 0) {  // x outside the sequence's steps: callers never ask for it
    r.j = 0;
    r.tile = 0;
    r.item_x0 = s_cum[lo];
    return r;
  }
  r.j = block_of_step(r.n_new, r.ctx, tq, p.window_left, off);
  const int before = steps_before_block(r.n_new, r.ctx, r.j, tq, p.window_left);
  r.item_x0 = s_cum[lo] + before;
  r.tile = block_tiles(r.n_new, r.ctx, r.j, tq, p.window_left).tile_lo + (off - before);
  return r;
}

__device__ __forceinline__ int unit_start_step(int total, int u, int units) {
  return static_cast<int>(static_cast<long long>(total) * u / units);
}

// 16 codes of an 8-bit cache row (one 16-byte chunk) -> 16 fp16 values times the row's scale, as two 16-byte groups.
// int8: (code ^ 0x80) under the exponent byte 0x64 is fp16 1152 + code, exactly; the packed subtract and multiply
// that follow are exact resp. correctly rounded.  fp8: the hardware conversion is exact.
template <int KIND>
__device__ __forceinline__ void dequant_chunk(uint4_t codes, float scale, uint4_t& lo, uint4_t& hi) {
  const _Float16 sh = static_cast<_Float16>(scale);
  const half2_t s2 = {sh, sh};
  uint32_t out[8];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t word = codes[w];
    half2_t a, c;
    if constexpr (KIND == KV_I8) {
      const uint32_t u = word ^ kI8Flip;
      const half2_t offs = {static_cast<_Float16>(kI8Offset), static_cast<_Float16>(kI8Offset)};
      a = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(kF16Filler, u, 0x04010400u)) - offs;
      c = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(kF16Filler, u, 0x04030402u)) - offs;
    } else {
      a = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, 1.0f, false));
      c = __builtin_bit_cast(half2_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(word, 1.0f, true));
    }
    out[2 * w] = __builtin_bit_cast(uint32_t, a * s2);
    out[2 * w + 1] = __builtin_bit_cast(uint32_t, c * s2);
  }
  lo = uint4_t{out[0], out[1], out[2], out[3]};
  hi = uint4_t{out[4], out[5], out[6], out[7]};
}

// DS > 1 (head dim 512): DS adjacent waves share a row tile, each with D / DS of the head's elements -- its part of
// K . Q^T, which the waves of the tile exchange through LDS and add in the same order, and its columns of O.
template <int KIND, int D, bool SCALE16, int RT, int DS = 1, bool ANYPAGE = false>
__global__ __launch_bounds__(kPrefillThreads, RT <= 2 ? 8 / kPrefillWaves : 1) void prefill_mfma_kernel(PrefillParams p) {
  static_assert(DS == 1 || RT == 1, "a split head has one row tile per wave group");
  constexpr int kRowTiles = RT;
  constexpr int kRowsPerWave = 16 * RT;  // rows of one wave (DS = 1) or of the DS waves that share them
  constexpr int kRowsPerWg = kRowsPerWave * kPrefillWaves / DS;
  constexpr int DW = D / DS;  // head-dim elements one wave multiplies and accumulates
  using T = KVTraits<KIND>;
  // The tiles in LDS are 16-bit whatever the cache holds: 8-bit codes are dequantized (times the per-token scale)
  // once, by the thread that stages them, instead of by every wave that reads them.
  constexpr int OPK = KIND == KV_BF16 ? KV_BF16 : KV_F16;
  using Ops = MfmaOps<OPK>;
  using V8 = typename Ops::vec8;
  using Pair = typename KVTraits<OPK>::pair_t;
  constexpr int ES = T::kBytes;  // bytes per element in the cache
  constexpr int EPL = 16 / ES;
  constexpr int LPT = D / EPL;  // 16-byte chunks per cached token row
  constexpr int TK = kTileTokens;
  constexpr int CHUNKS = TK * LPT;                                       // 16-byte chunks per cached K (or V) tile
  constexpr int NLD = (CHUNKS + kPrefillThreads - 1) / kPrefillThreads;  // loads per thread per tensor per tile
  constexpr int RSK = D * 2 + 16;
  constexpr int RSV = 2 * D + 32;
  constexpr int NS = DW / 32;
  constexpr int NB = DW / 16;
  typedef typename std::conditional<SCALE16, uint16_t, float>::type scale_raw_t;

  __shared__ __attribute__((aligned(16))) char s_k[2][TK * RSK];
  __shared__ __attribute__((aligned(16))) char s_v[2][TK * RSV];
  __shared__ int s_cum[kMaxPrefillSeqs + 1];
  __shared__ int s_wave_tot[kPrefillWaves];
  // score parts of a split head: [wave][tg][j][lane]
  __shared__ float s_part[DS > 1 ? kPrefillWaves : 1][2][4][DS > 1 ? kWave : 1];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lets the tile-level decisions stay scalar
  const int row_wave = wave / DS;  // which rows of the block the wave works on
  const int dpart = wave % DS;     // which part of the head dim
  const int d0 = dpart * DW;
  const int lr = lane & 15;
  const int lk = lane >> 4;
  // a kv head with more than 16 q heads runs as several "heads", each with up to 16 of them, that read the same K/V
  const int vhead = blockIdx.y;
  const int kvh = p.head_parts > 1 ? vhead / p.head_parts : vhead;
  const int head0 = kvh * p.group + 16 * (vhead - kvh * p.head_parts);   // first q head of this part
  const int group_here = min(16, (kvh + 1) * p.group - head0);           // q heads of this part
  const int vheads = p.kv_heads * p.head_parts;
  const int unit = blockIdx.x;
  const int tq = p.block_tokens;  // query tokens per item

  prefix_tile_steps(p, tq, s_cum, s_wave_tot);
  const int total = s_cum[p.num_seqs];
  const int x_begin = unit_start_step(total, unit, p.units);
  const int x_end = unit_start_step(total, unit + 1, p.units);
  if (x_begin >= x_end) return;  // same for the whole workgroup

  const bool q_is_operand_type = (OPK == KV_BF16 && p.q_dtype == ARENO_DT_BF16) ||
                                 (OPK == KV_F16 && p.q_dtype == ARENO_DT_F16);
  const bool packed = p.block_table == nullptr;  // K/V are (tokens, kv_heads, D): key t of a sequence is row q_begin + t
  constexpr int64_t row_bytes = static_cast<int64_t>(D) * ES;
  // A tile whose K and V chunks together are at most one per thread (8-bit tiles up to head dim 128, 16-bit ones at
  // 64) is staged with the workgroup split in two: the first half of the waves fetch, convert and publish K, the
  // second half V, one chunk per thread.  Otherwise every thread handles chunk i of K and of V for i < NLD, and for
  // such a tile the upper half of the workgroup would fetch clamped duplicates and publish nothing.
  constexpr bool kRoleSplit = 2 * CHUNKS <= kPrefillThreads;
  const bool role_v = kRoleSplit && wave >= kPrefillWaves / 2;  // wave-uniform
  // this thread's chunks of a tile: token and 16-byte column, fixed for the whole kernel
  int chunk_tok[NLD], chunk_col[NLD];
  bool chunk_live[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int c = (kRoleSplit && role_v ? tid - kPrefillThreads / 2 : tid) + kPrefillThreads * i;
    chunk_live[i] = (i + 1) * kPrefillThreads <= CHUNKS || c < CHUNKS;
    chunk_tok[i] = min(c, CHUNKS - 1) / LPT;
    chunk_col[i] = min(c, CHUNKS - 1) % LPT;
  }
  auto scale_value = [](scale_raw_t raw) -> float {
    if constexpr (SCALE16) {
      return static_cast<float>(__builtin_bit_cast(_Float16, raw));
    } else {
      return raw;
    }
  };

  StepPos pos = locate_step(p, s_cum, tq, x_begin);

  // What the staging steps ask block ids for: the item whose tiles are being fetched.  It is switched to the next
  // item before the current item's output is stored (see the end of the item loop).
  int fc_key_hi = 0, fc_q_begin = 0;
  const int32_t* fc_table_row = p.cu_seqlens_q;
  // ---- the tile pipeline -----------------------------------------------------------------------------------------
  // What one staging step fetches is published two steps later, so a fetch has two tile steps to arrive; block ids
  // are fetched two steps ahead of the chunk they locate.  Two sets of fetch registers alternate from step to step
  // (the tile loop is unrolled by two, so which set a step uses is fixed at compile time).
  struct FetchSet {
    int ids[NLD], keys[NLD];  // block id and key position of the tile to fetch next into this set
    uint4_t kreg[NLD], vreg[NLD];
    scale_raw_t ksreg[NLD], vsreg[NLD];
    uint32_t k_row[NLD];  // page row of the K chunk in this set: the V chunk of the same tile is fetched a step later
  };
  FetchSet set_a, set_b;
  {
    FetchSet zero;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      zero.ids[i] = zero.keys[i] = 0;
      zero.kreg[i] = zero.vreg[i] = uint4_t{0u, 0u, 0u, 0u};
      zero.ksreg[i] = zero.vsreg[i] = scale_raw_t(0);
      zero.k_row[i] = 0;
    }
    set_a = zero;
    set_b = zero;
  }
  // Addresses.  The cache row of key t is page_row * kv_heads + kvh with page_row = (block id << bs_shift) + t's slot
  // (packed K/V: q_begin + t), so a chunk's byte address is one 32 x 32 -> 64-bit multiply-add on a base that already
  // holds the pool, the head and the chunk's column (the launcher checks that page rows fit 32 bits).  The key a
  // block id was fetched for travels with the id.
  const uint32_t row_stride = static_cast<uint32_t>(p.kv_heads) * static_cast<uint32_t>(row_bytes);
  const uint32_t scale_stride = static_cast<uint32_t>(p.kv_heads) * static_cast<uint32_t>(sizeof(scale_raw_t));
  const uint32_t slot_mask = static_cast<uint32_t>(p.block_size - 1);
  auto chunk_base = [&](const void* pool, int i) {
    return static_cast<const char*>(pool) + static_cast<int64_t>(kvh) * row_bytes + chunk_col[i] * 16;
  };
  auto scale_base = [&](const void* pool) {
    return static_cast<const char*>(pool) + static_cast<int64_t>(kvh) * static_cast<int64_t>(sizeof(scale_raw_t));
  };
  auto chunk_at = [&](const char* base, uint32_t page_row) {
    return *reinterpret_cast<const uint4_t*>(base + static_cast<uint64_t>(page_row) * row_stride);
  };
  auto scale_at = [&](const char* base, uint32_t page_row) {
    return *reinterpret_cast<const scale_raw_t*>(base + static_cast<uint64_t>(page_row) * scale_stride);
  };
  // Page sizes that are no power of two have instances of their own (ANYPAGE; a choice at run time cost the
  // power-of-two instances 5 % of the launch): the key's column by a multiplication and a shift, the slot kept in
  // place of the key, the page row as a 24-bit multiply-add (the launcher checks the ranges).
  auto load_ids = [&](FetchSet& f, int tile) {
    int col[NLD];
    if constexpr (ANYPAGE) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int key = max(0, min(tile * TK + chunk_tok[i], fc_key_hi));
        col[i] = static_cast<int>(__umulhi(static_cast<uint32_t>(key), p.bs_magic) >> p.bs_post);
        f.keys[i] = key - __mul24(col[i], p.block_size);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int key = max(0, min(tile * TK + chunk_tok[i], fc_key_hi));
        f.keys[i] = packed ? fc_q_begin + key : key;  // packed K/V: the key's row itself
        col[i] = packed ? 0 : (key >> p.bs_shift);
      }
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) f.ids[i] = fc_table_row[col[i]];
  };
  // packed K/V run as one page per token with the token's row as its id
  auto page_row_of = [&](const FetchSet& f, int i) -> uint32_t {
    if constexpr (ANYPAGE) return static_cast<uint32_t>(__mul24(f.ids[i], p.block_size) + f.keys[i]);
    const uint32_t paged = (static_cast<uint32_t>(f.ids[i]) << p.bs_shift) + (static_cast<uint32_t>(f.keys[i]) & slot_mask);
    return packed ? static_cast<uint32_t>(f.keys[i]) : paged;
  };
  // The empty asm pins the use of a fetched chunk to this point of the iteration: without it the compiler converts
  // the codes right at the top of the loop and every tile waits there for the loads it has just issued.
  auto publish_k = [&](FetchSet& f, int tile) {
    char* kd = s_k[tile & 1];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      asm volatile("" : "+v"(f.kreg[i]));
      if (!chunk_live[i]) continue;
      const int t = chunk_tok[i];
      if constexpr (T::kQuant) {
        uint4_t lo, hi;
        dequant_chunk<KIND>(f.kreg[i], scale_value(f.ksreg[i]), lo, hi);
        char* kdst = kd + t * RSK + chunk_col[i] * 32;
        *reinterpret_cast<uint4_t*>(kdst) = lo;
        *reinterpret_cast<uint4_t*>(kdst + 16) = hi;
      } else {
        *reinterpret_cast<uint4_t*>(kd + t * RSK + chunk_col[i] * 16) = f.kreg[i];
      }
    }
  };
  auto publish_v = [&](FetchSet& f, int tile) {
    char* vd = s_v[tile & 1];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      asm volatile("" : "+v"(f.vreg[i]));
      if (!chunk_live[i]) continue;
      const int t = chunk_tok[i];
      if constexpr (T::kQuant) {
        uint4_t lo, hi;
        dequant_chunk<KIND>(f.vreg[i], scale_value(f.vsreg[i]), lo, hi);
        char* vdst = vd + v_row_of(t) * RSV + chunk_col[i] * 32;
        *reinterpret_cast<uint4_t*>(vdst) = lo;
        *reinterpret_cast<uint4_t*>(vdst + 16) = hi;
      } else {
        *reinterpret_cast<uint4_t*>(vd + v_row_of(t) * RSV + chunk_col[i] * 16) = f.vreg[i];
      }
    }
  };
  const char* const role_base = chunk_base(role_v ? p.v_cache : p.k_cache, 0);
  const char* const role_scale_base = scale_base(role_v ? p.v_scale : p.k_scale);
  // Staging step of iteration t with the fetch set `mine` of its parity (`other` is the previous and the next
  // step's): K[t + 2] and V[t + 1], fetched two steps ago, go from the registers into the LDS buffers the previous
  // iteration was the last to read; then K[t + 4] and V[t + 3] are fetched into the same registers, and the block
  // ids of K[t + 6] / V[t + 5].  It runs for every t (key positions are clamped into the item's range): tiles
  // outside [ta, tb] land in buffers nobody reads.
  auto stage = [&](int t, FetchSet& mine, FetchSet& other) {
    if constexpr (kRoleSplit) {
      // one chunk per thread: kreg / ksreg / ids hold the K chunk in a K wave and the V chunk in a V wave.  V runs
      // one tile behind K, as in the unsplit scheme.
      const int behind = role_v ? 1 : 0;
      asm volatile("" : "+v"(mine.kreg[0]));
      if (chunk_live[0]) {
        const int tk = chunk_tok[0];
        const int pub = t + 2 - behind;
        char* dst = role_v ? s_v[pub & 1] + v_row_of(tk) * RSV : s_k[pub & 1] + tk * RSK;
        if constexpr (T::kQuant) {
          uint4_t lo, hi;
          dequant_chunk<KIND>(mine.kreg[0], scale_value(mine.ksreg[0]), lo, hi);
          *reinterpret_cast<uint4_t*>(dst + chunk_col[0] * 32) = lo;
          *reinterpret_cast<uint4_t*>(dst + chunk_col[0] * 32 + 16) = hi;
        } else {
          *reinterpret_cast<uint4_t*>(dst + chunk_col[0] * 16) = mine.kreg[0];
        }
      }
      const uint32_t row = page_row_of(mine, 0);  // the ids of tile t + 4 - behind, fetched two steps ago
      mine.kreg[0] = chunk_at(role_base, row);
      if constexpr (T::kQuant) mine.ksreg[0] = scale_at(role_scale_base, row);
      load_ids(mine, t + 6 - behind);
    } else {
      publish_k(mine, t + 2);
      publish_v(mine, t + 1);
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        // V[t + 3]: the rows of K[t + 3], which the previous step fetched
        mine.vreg[i] = chunk_at(chunk_base(p.v_cache, i), other.k_row[i]);
        if constexpr (T::kQuant) mine.vsreg[i] = scale_at(scale_base(p.v_scale), other.k_row[i]);
      }
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const uint32_t row = page_row_of(mine, i);  // the ids of tile t + 4, fetched two steps ago
        mine.k_row[i] = row;
        mine.kreg[i] = chunk_at(chunk_base(p.k_cache, i), row);
        if constexpr (T::kQuant) mine.ksreg[i] = scale_at(scale_base(p.k_scale), row);
      }
      load_ids(mine, t + 6);
    }
  };


  // ---- the unit's segments ---------------------------------------------------------------------------------------
  // A segment is the part of an item (sequence, query block) inside the unit: key tiles [ta, tb].
  struct Segment {
    int seq, ta, tb, q_begin, ctx, tok0, tok_cnt;
    bool whole;  // the item's first and last tile are both here: its rows are final
  };
  auto segment_at = [&](const StepPos& q, int x_at) {
    const BlockTiles item = block_tiles(q.n_new, q.ctx, q.j, tq, p.window_left);
    Segment g;
    g.seq = q.seq;
    g.ta = q.tile;
    g.tb = min(item.tile_hi, q.tile + (x_end - x_at) - 1);
    g.whole = g.ta == item.tile_lo && g.tb == item.tile_hi;
    g.q_begin = q.q_begin;
    g.ctx = q.ctx;
    g.tok0 = item.tok0;
    g.tok_cnt = item.cnt;
    return g;
  };
  auto set_fetch_context = [&](const Segment& g) {
    fc_key_hi = g.ctx + g.tok0 + g.tok_cnt - 1;
    fc_q_begin = g.q_begin;
    // packed K/V have no table: the id load then reads a valid dummy word and its value is ignored
    fc_table_row = packed ? p.cu_seqlens_q : p.block_table + static_cast<int64_t>(g.seq) * p.max_blocks;
  };
  // the item behind q in the unit's order; false when the list is exhausted (cannot happen while the prefix sums and
  // this walk agree)
  auto next_position = [&](StepPos& q) -> bool {
    ++q.j;
    if (q.j * tq >= q.n_new) {
      q.j = 0;
      do {
        ++q.seq;
        if (q.seq >= p.num_seqs) return false;
        q.q_begin = p.cu_seqlens_q[q.seq];
        q.n_new = p.cu_seqlens_q[q.seq + 1] - q.q_begin;
      } while (q.n_new == 0);
      q.ctx = p.context_lens != nullptr ? p.context_lens[q.seq] : 0;
    }
    q.tile = block_tiles(q.n_new, q.ctx, q.j, tq, p.window_left).tile_lo;
    return true;
  };
  // ---- this lane's query rows: row R = wave * 16 RT + 16 * nq + lr -> token tok0 + R / fold, head R % fold ---------
  auto token_of_row = [&](int r) { return (r * p.fold_magic) >> 16; };
  int q_pos[kRowTiles];         // absolute position of the row's query, or -1 for a padding row
  int64_t row_elem[kRowTiles];  // element offset of the row in q / out
  V8 qop[kRowTiles][NS];
  auto load_q = [&](const Segment& g) {
#pragma unroll
    for (int nq = 0; nq < kRowTiles; ++nq) {
      const int r = row_wave * kRowsPerWave + 16 * nq + lr;
      const int t = token_of_row(r);
      const int hh = r - t * p.fold;
      const bool live = t < g.tok_cnt && hh < group_here;
      q_pos[nq] = live ? g.ctx + g.tok0 + t : -1;
      row_elem[nq] = (static_cast<int64_t>(g.q_begin + g.tok0 + t) * p.q_heads + head0 + hh) * D;
#pragma unroll
      for (int sl = 0; sl < NS; ++sl) {
        // (as fetched: a query of the other 16-bit type is converted behind the pipeline's fill, so that its fetch
        // and the fill's fetches are in flight together)
        uint4_t w = {0u, 0u, 0u, 0u};
        if (live) w = load16(p.q, (row_elem[nq] + d0 + (DW / 4) * lk + 8 * sl) * 2);
        qop[nq][sl] = __builtin_bit_cast(V8, w);
      }
    }
  };

  int x = x_begin;
  bool first_item = true;
  Segment seg = segment_at(pos, x);
  set_fetch_context(seg);
  load_q(seg);
  int prefilled = 0;  // staging steps of the segment's fill that ran before the previous segment's output was stored
  for (;;) {
    // ---- one segment: key tiles [ta, tb] of an item ------------------------------------------------------------------
    const int ta = seg.ta, tb = seg.tb;
    const bool whole = seg.whole;
    const int ctx = seg.ctx, tok0 = seg.tok0, tok_cnt = seg.tok_cnt;

    // rows of this wave: which query positions they span (wave-uniform), for skipping the mask on interior tiles
    const bool wave_live = row_wave * kRowsPerWave < tok_cnt * p.fold;
    const int wave_qmin = ctx + tok0 + token_of_row(row_wave * kRowsPerWave);
    const int wave_qmax = ctx + tok0 + min(tok_cnt - 1, token_of_row((row_wave + 1) * kRowsPerWave - 1));

    float4_t acc[kRowTiles][NB];
    // Row sums of the probabilities come from the matrix cores as well: one more product per key tile with an
    // all-ones A operand puts the sum over the tile's 32 keys of column (= query row) lr into every element of the
    // lane's accumulator, already complete over the four k groups.  Element 0 is the one kept (and rescaled).
    float4_t l_acc[kRowTiles];
    float m_run[kRowTiles];
    constexpr uint32_t kOnePair = OPK == KV_BF16 ? 0x3f803f80u : 0x3c003c00u;  // two 1.0 in the operand type
    const V8 ones_op = __builtin_bit_cast(V8, uint4_t{kOnePair, kOnePair, kOnePair, kOnePair});
#pragma unroll
    for (int nq = 0; nq < kRowTiles; ++nq) {
      m_run[nq] = kNegInf;
      l_acc[nq] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nq][nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // raw scores of one key tile: S^T = K . Q^T
    float s_cur[kRowTiles][2][4];
    auto scores = [&](int tile, float (&s)[kRowTiles][2][4]) {
      const char* kt = s_k[tile & 1];
#pragma unroll
      for (int tg = 0; tg < 2; ++tg) {
        const char* krow = kt + (16 * tg + lr) * RSK + (d0 + (DW / 4) * lk) * 2;
        V8 kop[NS];
#pragma unroll
        for (int sl = 0; sl < NS; ++sl) kop[sl] = *reinterpret_cast<const V8*>(krow + 16 * sl);
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) {
          float4_t c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int sl = 0; sl < NS; ++sl) c = Ops::mfma(kop[sl], qop[nq][sl], c);
#pragma unroll
          for (int j = 0; j < 4; ++j) s[nq][tg][j] = c[j];
        }
      }
    };

    // ---- fill the pipe: after these iterations K[ta], K[ta + 1] and V[ta] are in LDS (the first ones only fetch) ------
    for (int t = ta - 6 + prefilled; t < ta; t += 2) {
      lds_barrier();
      stage(t, set_a, set_b);
      lds_barrier();
      stage(t + 1, set_b, set_a);
    }
    lds_barrier();
    if (!q_is_operand_type) {
#pragma unroll
      for (int nq = 0; nq < kRowTiles; ++nq) {
#pragma unroll
        for (int sl = 0; sl < NS; ++sl) {
          uint4_t w = __builtin_bit_cast(uint4_t, qop[nq][sl]);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t word = w[j];
            float a, c;
            if constexpr (OPK == KV_BF16) {
              a = f16_bits_to_float(word & 0xffffu);
              c = f16_bits_to_float(word >> 16);
            } else {
              a = bf16_bits_to_float(word & 0xffffu);
              c = bf16_bits_to_float(word >> 16);
            }
            w[j] = __builtin_bit_cast(uint32_t, make_pair<Pair>(a, c));
          }
          qop[nq][sl] = __builtin_bit_cast(V8, w);
        }
      }
    }
    if (DS == 1 && wave_live) scores(ta, s_cur);

    // ---- iteration t: staging first, then the scores of tile t + 1 go to the matrix cores in the same block as the row
    // maxima of tile t ---------------------------------------------------------------------------------------------------
    // One tile step is a lambda over (scores of tile t, room for the scores of tile t + 1) and the loop calls it twice
    // with the two arrays swapped: the scores of the next tile are then computed where the following step reads them
    // and no per-tile register copy of the 8 * kRowTiles scores is left.
    float s_alt[kRowTiles][2][4];
    auto tile_step = [&](int t, float (&s_cur)[kRowTiles][2][4], float (&s_next)[kRowTiles][2][4], FetchSet& mine,
                         FetchSet& other) {
      lds_barrier();
      if constexpr (DS == 1) stage(t, mine, other);
      if constexpr (DS > 1) {
        // A split head computes the scores of tile t here (K[t] was published two steps ago), hands its part to the
        // other waves of its rows and adds all parts in index order, so that those waves go on with identical scores.
        // The staging step, which overwrites K[t] with K[t + 2], comes behind the second barrier, when every wave has
        // read K[t]; the parts are read before the next step's barrier, which is what lets one buffer do.  (No
        // overlap of these products with the previous tile's softmax, and a second barrier per tile: the price of
        // the wide head.)
        if (wave_live) {
          scores(t, s_cur);
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) s_part[wave][tg][j][lane] = s_cur[0][tg][j];
          }
        }
        lds_barrier();
        stage(t, mine, other);
        if (wave_live) {
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float sum = s_part[row_wave * DS][tg][j][lane];
#pragma unroll
              for (int part = 1; part < DS; ++part) sum += s_part[row_wave * DS + part][tg][j][lane];
              s_cur[0][tg][j] = sum;
            }
          }
        }
      }
      if (!wave_live) return;
      const int k0 = t * TK;
      const bool need_mask = k0 + TK - 1 > wave_qmin || (p.window_left >= 0 && k0 < wave_qmax - p.window_left);
      if (need_mask) {
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) {
          // key 16 tg + j of this lane's 4-key groups is visible iff its index is <= hi (causal) and >= hi - window
          const int hi = q_pos[nq] - k0 - 4 * lk;
          if (p.window_left < 0) {
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
              for (int j = 0; j < 4; ++j) s_cur[nq][tg][j] = 16 * tg + j <= hi ? s_cur[nq][tg][j] : kNegInf;
            }
          } else {
            const int lo = hi - p.window_left;
            const uint32_t span = static_cast<uint32_t>(p.window_left);
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const bool ok = static_cast<uint32_t>(16 * tg + j - lo) <= span;  // 0 <= index - lo <= window
                s_cur[nq][tg][j] = ok ? s_cur[nq][tg][j] : kNegInf;
              }
            }
          }
        }
      }
      if constexpr (DS == 1) scores(t + 1, s_next);  // past tb this reads a buffer of clamped or stale keys; the result is dropped
      // -- online softmax in the log2 domain; the (positive) softmax scale is applied to the row maximum and inside
      // the exponent's multiply-add -----------------------------------------------------------------------------------
      // The reference value m of a row only has to be the same for all its keys and to bound the scores well enough
      // for the exponentials to fit the operand type; it need not be the exact maximum.  So it is raised (and the
      // accumulators rescaled) only when a tile's scores exceed it by more than kLazy in the log2 domain (a factor
      // 2^kLazy in the probabilities, far inside fp16's range); each lane checks its own eight scores and one ballot
      // decides for the wave, which skips the cross-lane maximum and the rescale on most tiles.
      constexpr float kLazy = 8.0f;
      float mt_lane[kRowTiles];
      bool raise = false;
#pragma unroll
      for (int nq = 0; nq < kRowTiles; ++nq) {
        mt_lane[nq] = max3_f32(max3_f32(s_cur[nq][0][0], s_cur[nq][0][1], s_cur[nq][0][2]),
                               max3_f32(s_cur[nq][0][3], s_cur[nq][1][0], s_cur[nq][1][1]),
                               max3_f32(s_cur[nq][1][2], s_cur[nq][1][3], s_cur[nq][1][3]));
        // (-inf > -inf + kLazy is false: a fully masked row stays at -inf; anything finite beats -inf)
        raise = raise | (mt_lane[nq] * p.scale_log2e > m_run[nq] + kLazy);  // no short circuit: straight-line code
      }
      if (__builtin_amdgcn_ballot_w64(raise) != 0) {
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) {
          const float mt = rows_max(mt_lane[nq]) * p.scale_log2e;
          const float m_new = max_f32(m_run[nq], mt);
          const float m_ref = m_new == kNegInf ? 0.0f : m_new;
          const float alpha = settled(fast_exp2(m_run[nq] - m_ref));
          m_run[nq] = m_new;
          {
            float l0 = l_acc[nq][0];
            scale_in_place(l0, alpha);
            l_acc[nq][0] = l0;
          }
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float a = acc[nq][nb][j];
              scale_in_place(a, alpha);
              acc[nq][nb][j] = a;
            }
          }
        }
      }
      float m_safe[kRowTiles];
#pragma unroll
      for (int nq = 0; nq < kRowTiles; ++nq) m_safe[nq] = m_run[nq] == kNegInf ? 0.0f : m_run[nq];
      V8 pop[kRowTiles];
#pragma unroll
      for (int nq = 0; nq < kRowTiles; ++nq) {
        float pe[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pe[j] = fast_exp2(__builtin_fmaf(s_cur[nq][0][j], p.scale_log2e, -m_safe[nq]));
          pe[4 + j] = fast_exp2(__builtin_fmaf(s_cur[nq][1][j], p.scale_log2e, -m_safe[nq]));
        }
        uint32_t pw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pw[j] = pack_pair<OPK>(pe[2 * j], pe[2 * j + 1]);
        pop[nq] = __builtin_bit_cast(V8, uint4_t{pw[0], pw[1], pw[2], pw[3]});
        l_acc[nq] = Ops::mfma(ones_op, pop[nq], l_acc[nq]);  // sums the probabilities as rounded for the product
      }

      // -- O^T += V^T . P^T: lane i of a 16-lane group supplies row (i / 4), 4 elements at column 16 nb + 4 (i % 4);
      // two transpose reads of 4 tokens each -----------------------------------------------------------------------------
      char* vt = s_v[t & 1];
      const int r4 = lr >> 2;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        uint32_t vw[4];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int tok = 16 * half + 4 * lk + r4;
          char* a = vt + v_row_of(tok) * RSV + (d0 + 16 * nb + 4 * (lr & 3)) * 2;
          const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
          const uint2_t u = __builtin_bit_cast(uint2_t, r);
          vw[2 * half] = u[0];
          vw[2 * half + 1] = u[1];
        }
        const V8 vop = __builtin_bit_cast(V8, uint4_t{vw[0], vw[1], vw[2], vw[3]});
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) acc[nq][nb] = Ops::mfma(vop, pop[nq], acc[nq][nb]);
      }
    };
    for (int t = ta; t <= tb; t += 2) {
      tile_step(t, s_cur, s_alt, set_a, set_b);
      if (t + 1 > tb) break;
      tile_step(t + 1, s_alt, s_cur, set_b, set_a);
    }

    // ---- the next segment's first fetches go out in front of this segment's output -------------------------------
    // The memory queue retires in order: whatever is fetched behind the output stores is waited for together with
    // their acknowledgement (~3 us).  So the next segment's query rows and the block ids of its first two tiles (the
    // first two steps of its fill) are requested here, and the rest of its fill runs while the stores drain.
    x += tb - ta + 1;
    const bool more = x < x_end && next_position(pos);
    int done_q_pos[kRowTiles];
    int64_t done_row_elem[kRowTiles];
#pragma unroll
    for (int nq = 0; nq < kRowTiles; ++nq) {
      done_q_pos[nq] = q_pos[nq];
      done_row_elem[nq] = row_elem[nq];
    }
    if (more) {
      seg = segment_at(pos, x);
      set_fetch_context(seg);
      lds_barrier();  // every wave has left this segment's tiles (only LDS needs ordering here)
      stage(seg.ta - 6, set_a, set_b);
      lds_barrier();
      stage(seg.ta - 5, set_b, set_a);
      load_q(seg);
    }

    // ---- finish the segment: final rows go to `out`, a cut item leaves its partial in the workspace ---------------
    const int slot = 2 * unit + (first_item ? 0 : 1);
#pragma unroll
    for (int nq = 0; nq < kRowTiles; ++nq) {
      const float l_tot = l_acc[nq][0];
      if (done_q_pos[nq] < 0) continue;
      if (whole) {
        const float inv = 1.0f / l_tot;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int64_t e0 = done_row_elem[nq] + d0 + 16 * nb + 4 * lk;
          uint32_t lo, hi;
          const float o0 = acc[nq][nb][0] * inv, o1 = acc[nq][nb][1] * inv;
          const float o2 = acc[nq][nb][2] * inv, o3 = acc[nq][nb][3] * inv;
          if (p.q_dtype == ARENO_DT_BF16) {
            lo = float_to_bf16_bits(o0) | (float_to_bf16_bits(o1) << 16);
            hi = float_to_bf16_bits(o2) | (float_to_bf16_bits(o3) << 16);
          } else {
            lo = float_to_f16_bits(o0) | (float_to_f16_bits(o1) << 16);
            hi = float_to_f16_bits(o2) | (float_to_f16_bits(o3) << 16);
          }
          *reinterpret_cast<uint2_t*>(static_cast<char*>(p.out) + e0 * 2) = uint2_t{lo, hi};
        }
      } else {
        const int r = row_wave * kRowsPerWave + 16 * nq + lr;
        const int64_t prow = (static_cast<int64_t>(slot) * vheads + vhead) * kRowsPerWg + r;
        float* dst = p.part_acc + prow * D + d0 + 4 * lk;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) *reinterpret_cast<float4_t*>(dst + 16 * nb) = acc[nq][nb];
        if (lk == 0 && dpart == 0) {
          p.part_ml[prow * 2] = m_run[nq];
          p.part_ml[prow * 2 + 1] = l_tot;
        }
      }
    }

    first_item = false;
    if (!more) break;
    prefilled = 2;
  }
}

// Merge of the items cut by unit borders.  Workgroup (u, kv head) looks at the last item of unit u: if that item
// starts in unit u and runs on into later units, it combines the partials of all units the item touches (slot
// 2u' for a unit where the item comes first, 2u' + 1 where it comes last after other items), normalises and
// writes the item's rows.
constexpr int kMergeInFlight = 8;  // 16-byte chunks of each partial a thread of prefill_merge_kernel takes

__global__ __launch_bounds__(kPrefillThreads) void prefill_merge_kernel(PrefillParams p) {
  __shared__ int s_cum[kMaxPrefillSeqs + 1];
  __shared__ int s_wave_tot[kPrefillWaves];
  const int tid = threadIdx.x;
  const int unit = blockIdx.x;
  const int vhead = blockIdx.y;
  const int kvh = p.head_parts > 1 ? vhead / p.head_parts : vhead;
  const int head0 = kvh * p.group + 16 * (vhead - kvh * p.head_parts);
  const int group_here = min(16, (kvh + 1) * p.group - head0);
  const int vheads = p.kv_heads * p.head_parts;
  const int kRowsPerWg = p.rows_per_wg;
  const int tq = p.block_tokens;
  const int d = p.head_dim;
  prefix_tile_steps(p, tq, s_cum, s_wave_tot);
  const int total = s_cum[p.num_seqs];
  const int x_begin = unit_start_step(total, unit, p.units);
  const int x_end = unit_start_step(total, unit + 1, p.units);
  if (x_begin >= x_end) return;
  const StepPos pos = locate_step(p, s_cum, tq, x_end - 1);
  const BlockTiles item = block_tiles(pos.n_new, pos.ctx, pos.j, tq, p.window_left);
  const int item_x1 = pos.item_x0 + item.count();
  if (item_x1 <= x_end || pos.item_x0 < x_begin) return;  // not cut here, or merged by the unit where it starts
  // last unit that owns a step of the item: the largest u with unit_start_step(u) <= item_x1 - 1
  int u_hi = static_cast<int>((static_cast<long long>(item_x1) * p.units - 1) / total);
  if (u_hi > p.units - 1) u_hi = p.units - 1;
  while (unit_start_step(total, u_hi, p.units) > item_x1 - 1) --u_hi;
  while (u_hi + 1 < p.units && unit_start_step(total, u_hi + 1, p.units) <= item_x1 - 1) ++u_hi;

  const int q_begin = pos.q_begin;
  // The partials of a slot are one contiguous block of rows x head_dim floats, walked as a flat array of 16-byte
  // chunks, consecutive threads on consecutive chunks (a thread per row part left three quarters of every fetched
  // line to a later instruction).  The kernel is a chain of dependent round trips on one workgroup per CU, so the
  // chain is kept short: a workgroup takes kInFlight chunks per thread of every partial (blockIdx.z picks which; the
  // launcher sizes the grid), the partials are combined in one pass with a running maximum, and the fetches of the
  // next partial are issued before the current one is used.  (One workgroup per cut item walking all chunks in two
  // passes took 32 us for the ~500 partials of a launch, 2.1 TB/s.)  The (m, l) pair of a chunk's row is the same
  // for the lanes of the row and comes out of the cache.
  const int chunks_per_row = d >> 2;
  const int total_chunks = kRowsPerWg * chunks_per_row;
  const float inv_chunks_per_row = 1.0f / static_cast<float>(chunks_per_row);
  const int base = blockIdx.z * kMergeInFlight * kPrefillThreads + tid;
  if (base >= total_chunks) return;
  {
    constexpr int kInFlight = kMergeInFlight;
    int row[kInFlight];
    bool live[kInFlight];
    float m[kInFlight], lsum[kInFlight];
    float4_t o[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      const int idx = min(base + k * kPrefillThreads, total_chunks - 1);
      // idx / chunks_per_row: the product with the rounded reciprocal is exact here (idx + 0.5 is at least half a
      // chunk away from a multiple of chunks_per_row, and idx < 2^16)
      row[k] = static_cast<int>((static_cast<float>(idx) + 0.5f) * inv_chunks_per_row);
      const int t = (row[k] * p.fold_magic) >> 16;
      const int hh = row[k] - t * p.fold;
      live[k] = base + k * kPrefillThreads < total_chunks && t < item.cnt && hh < group_here;
      m[k] = kNegInf;
      lsum[k] = 0.0f;
      o[k] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    struct Fetched {
      float4_t a[kInFlight];
      float2_t v[kInFlight];
    };
    auto next_unit = [&](int u) {  // the next unit from u on that owns steps, or u_hi + 1
      while (u <= u_hi && unit_start_step(total, u, p.units) == unit_start_step(total, u + 1, p.units)) ++u;
      return u;
    };
    auto fetch = [&](Fetched& f, int u) {
      const int slot = 2 * u + ((u == unit && pos.item_x0 > x_begin) ? 1 : 0);
      const int64_t slot_row0 = (static_cast<int64_t>(slot) * vheads + vhead) * kRowsPerWg;
      const float* ml = p.part_ml + slot_row0 * 2;
      const float4_t* acc = reinterpret_cast<const float4_t*>(p.part_acc + slot_row0 * d);
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) {
        f.a[k] = acc[min(base + k * kPrefillThreads, total_chunks - 1)];
        f.v[k] = *reinterpret_cast<const float2_t*>(ml + 2 * row[k]);
      }
    };
    Fetched cur, nxt;
    int u = next_unit(unit);  // (unit itself owns steps: checked above)
    fetch(cur, u);
    for (;;) {
      const int u2 = next_unit(u + 1);
      if (u2 <= u_hi) fetch(nxt, u2);
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) {
        if (cur.v[k][1] == 0.0f) continue;  // a partial without visible keys contributes nothing
        const float m_new = fmaxf(m[k], cur.v[k][0]);
        const float keep = fast_exp2(m[k] - m_new);  // 0 for the first partial (m = -inf)
        const float w = fast_exp2(cur.v[k][0] - m_new);
        lsum[k] = lsum[k] * keep + w * cur.v[k][1];
#pragma unroll
        for (int j = 0; j < 4; ++j) o[k][j] = o[k][j] * keep + w * cur.a[k][j];
        m[k] = m_new;
      }
      if (u2 > u_hi) break;
      cur = nxt;
      u = u2;
    }
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      if (!live[k]) continue;
      const int idx = base + k * kPrefillThreads;
      const int t = (row[k] * p.fold_magic) >> 16;
      const int hh = row[k] - t * p.fold;
      const float inv = 1.0f / lsum[k];
      const int64_t out_elem = (static_cast<int64_t>(q_begin + item.tok0 + t) * p.q_heads + head0 + hh) * d +
                               4 * (idx - row[k] * chunks_per_row);
      uint32_t lo, hi;
      if (p.q_dtype == ARENO_DT_BF16) {
        lo = float_to_bf16_bits(o[k][0] * inv) | (float_to_bf16_bits(o[k][1] * inv) << 16);
        hi = float_to_bf16_bits(o[k][2] * inv) | (float_to_bf16_bits(o[k][3] * inv) << 16);
      } else {
        lo = float_to_f16_bits(o[k][0] * inv) | (float_to_f16_bits(o[k][1] * inv) << 16);
        hi = float_to_f16_bits(o[k][2] * inv) | (float_to_f16_bits(o[k][3] * inv) << 16);
      }
      *reinterpret_cast<uint2_t*>(static_cast<char*>(p.out) + out_elem * 2) = uint2_t{lo, hi};
    }
  }
}

typedef void (*prefill_fn)(PrefillParams);

template <int KIND, int RT, bool ANYPAGE>
prefill_fn prefill_lookup_rt(int head_dim, bool scale16) {
  constexpr bool kQuant = KVTraits<KIND>::kQuant;
  if constexpr (RT == 2) {
    if (head_dim == 128) {
      if constexpr (kQuant) {
        if (scale16) return prefill_mfma_kernel<KIND, 128, true, 2, 1, ANYPAGE>;
      }
      return prefill_mfma_kernel<KIND, 128, false, 2, 1, ANYPAGE>;
    }
    if (head_dim == 64) {
      if constexpr (kQuant) {
        if (scale16) return prefill_mfma_kernel<KIND, 64, true, 2, 1, ANYPAGE>;
      }
      return prefill_mfma_kernel<KIND, 64, false, 2, 1, ANYPAGE>;
    }
  } else {
    if (head_dim == 256) {
      if constexpr (kQuant) {
        if (scale16) return prefill_mfma_kernel<KIND, 256, true, 1, 1, ANYPAGE>;
      }
      return prefill_mfma_kernel<KIND, 256, false, 1, 1, ANYPAGE>;
    }
    if (head_dim == 192) {
      if constexpr (kQuant) {
        if (scale16) return prefill_mfma_kernel<KIND, 192, true, 1, 1, ANYPAGE>;
      }
      return prefill_mfma_kernel<KIND, 192, false, 1, 1, ANYPAGE>;
    }
    if (head_dim == 512) {
      if constexpr (kQuant) {
        if (scale16) return prefill_mfma_kernel<KIND, 512, true, 1, 2, ANYPAGE>;
      }
      return prefill_mfma_kernel<KIND, 512, false, 1, 2, ANYPAGE>;
    }
  }
  return nullptr;
}

// 16-row tiles per wave: two up to head dim 128 (four need more registers than a wave has), one at head dims 192 and
// 256, where the accumulators and the Q operands of one tile take the registers two take at 128; at 512 two waves
// share a tile, 256 elements each.
int prefill_row_tiles(int head_dim) { return head_dim > 128 ? 1 : 2; }
int prefill_head_split(int head_dim) { return head_dim > 256 ? 2 : 1; }
int prefill_rows_per_wg(int head_dim) { return 16 * prefill_row_tiles(head_dim) * kPrefillWaves / prefill_head_split(head_dim); }

template <int KIND>
prefill_fn prefill_lookup(int head_dim, bool scale16, int row_tiles, bool any_page_size) {
  if (any_page_size)
    return row_tiles == 1 ? prefill_lookup_rt<KIND, 1, true>(head_dim, scale16) : prefill_lookup_rt<KIND, 2, true>(head_dim, scale16);
  return row_tiles == 1 ? prefill_lookup_rt<KIND, 1, false>(head_dim, scale16) : prefill_lookup_rt<KIND, 2, false>(head_dim, scale16);
}

int log2_exact_i(int x) {
  if (x <= 0 || (x & (x - 1)) != 0) return -1;
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}

int prefill_units(int kv_heads) {
  int u = kPrefillTargetWgs / kv_heads;
  if (u < 1) u = 1;
  if (u > kMaxPrefillUnits) u = kMaxPrefillUnits;
  return u;
}

size_t prefill_ml_bytes(int units, int kv_heads) {
  return static_cast<size_t>(2) * units * kv_heads * kMaxRowsPerWg * 2 * sizeof(float);
}

}  // namespace

size_t prefill_mfma_workspace_bytes(int32_t kv_heads, int32_t head_dim) {
  if (kv_heads <= 0 || head_dim <= 0) return 0;
  const int units = prefill_units(kv_heads);
  return prefill_ml_bytes(units, kv_heads) +
         static_cast<size_t>(2) * units * kv_heads * prefill_rows_per_wg(head_dim) * head_dim * sizeof(float);
}

// block_table == nullptr selects packed K/V: cache->k / cache->v then point at (tokens, kv_heads, D) tensors and
// context_lens may be nullptr (no cached context).
int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* workspace, size_t workspace_bytes, void* stream) {
  const char* op = "areno_hip_paged_varlen_prefill";
  const int group = q_heads / cache->kv_heads;
  if (q_dtype != ARENO_DT_F16 && q_dtype != ARENO_DT_BF16) return ARENO_ERR_UNSUPPORTED;
  if (!(softmax_scale > 0.0f)) return ARENO_ERR_UNSUPPORTED;  // the kernel takes row maxima before scaling
  // page addressing by shift and mask, or, for page sizes that are no power of two, by a multiplication and a shift
  // (keys below 2^30) and 24-bit products (block ids, table columns and page sizes below 2^23)
  const bool pow2_pages = log2_exact_i(cache->block_size) >= 0;
  PageDivision division = {0, 0};
  if (!pow2_pages) {
    if (block_table == nullptr || !page_division(cache->block_size, &division)) return ARENO_ERR_UNSUPPORTED;
    if (cache->num_blocks >= (1 << 23) || cache->block_size >= (1 << 23) || max_blocks >= (1 << 23) ||
        static_cast<int64_t>(max_blocks) * cache->block_size > 0x3fffffffLL)
      return ARENO_ERR_UNSUPPORTED;
  }
  const int head_parts = (group + 15) / 16;
  const int vheads = cache->kv_heads * head_parts;
  if (head_parts > 8 || num_seqs > kMaxPrefillSeqs || tokens > 0x3fffffff) return ARENO_ERR_UNSUPPORTED;
  if (vheads > 65535) return ARENO_ERR_UNSUPPORTED;
  // page rows (block id * page size + slot, or token rows of packed K/V) are 32-bit in the kernel's address arithmetic
  if (block_table != nullptr && cache->num_blocks * cache->block_size > 0xffffffffLL) return ARENO_ERR_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(cache->k) % 16 != 0 || reinterpret_cast<uintptr_t>(cache->v) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(q) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 8 != 0)
    return ARENO_ERR_UNSUPPORTED;
  const bool scale16 = cache->scale_dtype == ARENO_DT_F16;
  const int row_tiles = prefill_row_tiles(cache->head_dim);
  const int rows_per_wg = prefill_rows_per_wg(cache->head_dim);
  prefill_fn fn = nullptr;
  switch (cache->cache_dtype) {
    case ARENO_DT_BF16: fn = prefill_lookup<KV_BF16>(cache->head_dim, scale16, row_tiles, !pow2_pages); break;
    case ARENO_DT_F16: fn = prefill_lookup<KV_F16>(cache->head_dim, scale16, row_tiles, !pow2_pages); break;
    case ARENO_DT_I8: fn = prefill_lookup<KV_I8>(cache->head_dim, scale16, row_tiles, !pow2_pages); break;
    case ARENO_DT_FP8_E4M3: fn = prefill_lookup<KV_FP8>(cache->head_dim, scale16, row_tiles, !pow2_pages); break;
    default: break;
  }
  if (fn == nullptr) return ARENO_ERR_UNSUPPORTED;
  // tile steps are counted in 32-bit: (tokens / query block + seqs) * (longest visible range / 32) must fit; the
  // paged case is bounded by the table width
  const int64_t max_keys = block_table != nullptr ? static_cast<int64_t>(max_blocks) * cache->block_size : tokens;
  const int fold = head_parts > 1 ? 16 : group;  // rows of a token in a query block
  const int block_tokens = rows_per_wg / fold;
  {
    const int64_t items = tokens / block_tokens + num_seqs;
    if (items * (max_keys / kTileTokens + 1) > 0x7fffffffLL) return ARENO_ERR_UNSUPPORTED;
  }
  // (the partials of a launch laid out over (kv head, part) pairs never need more than the kv heads alone would,
  // except when the pairs outnumber the launch's workgroups: then the generic kernel takes the call)
  const size_t need = prefill_mfma_workspace_bytes(cache->kv_heads, cache->head_dim);
  if (head_parts > 1 && prefill_mfma_workspace_bytes(vheads, cache->head_dim) > need) return ARENO_ERR_UNSUPPORTED;
  if (workspace == nullptr || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
    return fail(ARENO_ERR_WORKSPACE, "%s: workspace of %zu bytes (16-byte aligned) required, got %zu", op, need,
                workspace_bytes);

  PrefillParams p;
  p.q = q;
  p.out = out;
  p.k_cache = cache->k;
  p.v_cache = cache->v;
  p.k_scale = cache->k_scale;
  p.v_scale = cache->v_scale;
  p.block_table = block_table;
  p.cu_seqlens_q = cu_seqlens_q;
  p.context_lens = context_lens;
  p.num_seqs = num_seqs;
  p.q_heads = q_heads;
  p.kv_heads = cache->kv_heads;
  p.head_dim = cache->head_dim;
  p.group = group;
  p.head_parts = head_parts;
  p.fold = fold;
  p.fold_magic = (65536 + fold - 1) / fold;
  p.block_tokens = block_tokens;
  p.block_size = cache->block_size;
  p.bs_shift = log2_exact_i(cache->block_size);
  p.bs_magic = division.magic;
  p.bs_post = division.post;
  p.max_blocks = max_blocks;
  p.window_left = window_left;
  p.q_dtype = q_dtype;
  p.units = prefill_units(vheads);
  p.rows_per_wg = rows_per_wg;
  p.scale_log2e = softmax_scale * kLog2e;
  p.part_ml = static_cast<float*>(workspace);
  p.part_acc = reinterpret_cast<float*>(static_cast<char*>(workspace) + prefill_ml_bytes(p.units, vheads));
  const dim3 grid(p.units, vheads);
  hipLaunchKernelGGL(fn, grid, dim3(kPrefillThreads), 0, static_cast<hipStream_t>(stream), p);
  if (int rc = check_launch(op)) return rc;
  const int merge_parts = (rows_per_wg * (cache->head_dim / 4) + kMergeInFlight * kPrefillThreads - 1) / (kMergeInFlight * kPrefillThreads);
  hipLaunchKernelGGL(prefill_merge_kernel, dim3(p.units, vheads, merge_parts), dim3(kPrefillThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}

}  // namespace areno
