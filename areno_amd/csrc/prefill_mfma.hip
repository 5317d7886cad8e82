// Causal varlen prefill over paged (optionally quantized) KV on the matrix cores (gfx950).
//
// Workgroup = 4 wave64 = one (sequence, kv head, block of query tokens).  The G query heads of the kv head
// are folded into the query-row axis: row r of the block is (token r / GP, head r % GP) with GP = G rounded up
// to a power of two, so one 16-row MFMA tile holds 16 / GP tokens of all heads and K/V are read once for the
// whole group (GQA without expanding KV, as areno/accel/csrc/attention.cu:170-171 does per row).
// Each wave owns 32 query rows (two 16-row tiles); the workgroup walks the visible keys in 32-token tiles:
//   * all 256 threads fetch the next K/V tile with 16-byte coalesced loads (block ids resolved one tile ahead)
//     while the current tile is computed, then store it into a shared LDS tile (padded rows, conflict free);
//   * S^T[key][row] = K . Q^T   : A = K rows from LDS, B = Q^T in registers; C has row = lane % 16, 4 keys per lane;
//   * causal / window / length mask, per-key K scale, online softmax in the log2 domain (per lane = per row);
//   * O^T[dim][row] += V^T . P^T : A = V^T through the LDS transpose reads, B = P^T (= the C layout of S^T).
// The dequantisation of int8 / fp8 codes and the layouts are the ones of the decode kernel
// (decode_mfma_kernels.hpp).  Semantics: _reference_attention with query_start = context_lens[s]
// (areno/accel/attention.py:25-41 in the reference); with context 0 it is the reference's varlen kernel
// (areno/accel/csrc/attention.cu:145-242).

#include "decode_mfma_kernels.hpp"

namespace areno {

int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* stream);

namespace {

constexpr int kPrefillThreads = 256;
constexpr int kPrefillWaves = 4;
constexpr int kRowTiles = 2;                          // 16-row MFMA tiles per wave
constexpr int kRowsPerWave = 16 * kRowTiles;          // 32
constexpr int kRowsPerWg = kRowsPerWave * kPrefillWaves;  // 128
constexpr int kMaxPrefillSeqs = 1024;

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
  int32_t num_seqs;
  int32_t q_heads;
  int32_t kv_heads;
  int32_t group;         // q heads per kv head
  int32_t group_pad;     // rounded up to a power of two (<= 16)
  int32_t group_shift;   // log2(group_pad)
  int32_t block_size;
  int32_t bs_shift;
  int32_t max_blocks;
  int32_t window_left;
  int32_t q_dtype;
  float scale_log2e;
};

template <int KIND, int D, bool SCALE16>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_mfma_kernel(PrefillParams p) {
  using T = KVTraits<KIND>;
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using Pair = typename T::pair_t;
  constexpr int ES = T::kBytes;
  constexpr int EPL = 16 / ES;
  constexpr int LPT = D / EPL;  // 16-byte chunks per token row
  constexpr int TK = kTileTokens;
  constexpr int CHUNKS = TK * LPT;                   // 16-byte chunks per K (or V) tile
  constexpr int NLD = (CHUNKS + kPrefillThreads - 1) / kPrefillThreads;  // loads per thread per tensor per tile
  constexpr int RSK = D * ES + 16;
  constexpr int RSV = ES == 1 ? D + 16 : 2 * D + 32;
  constexpr int NS = D / 32;
  constexpr int NB = D / 16;
  constexpr int WPL = 8 * ES / 4;
  constexpr float kPScale = T::kQuant ? 256.0f : 1.0f;
  typedef typename std::conditional<SCALE16, uint16_t, float>::type scale_raw_t;

  __shared__ __attribute__((aligned(16))) char s_k[TK * RSK];
  __shared__ __attribute__((aligned(16))) char s_v[TK * RSV];
  __shared__ float s_ksc[TK];
  __shared__ float s_vsc[TK];
  __shared__ int s_cum[kMaxPrefillSeqs + 1];
  __shared__ int s_wave_tot[kPrefillWaves];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int lr = lane & 15;
  const int lk = lane >> 4;
  const int kvh = blockIdx.y;
  const int tokens_per_wg = kRowsPerWg >> p.group_shift;

  // ---- which (sequence, query block) is this workgroup?  prefix sum of blocks per sequence ---------------
  {
    constexpr int SPT = kMaxPrefillSeqs / kPrefillThreads;
    int nb[SPT];
    int local = 0;
#pragma unroll
    for (int j = 0; j < SPT; ++j) {
      const int s = SPT * tid + j;
      nb[j] = 0;
      if (s < p.num_seqs) nb[j] = (p.cu_seqlens_q[s + 1] - p.cu_seqlens_q[s] + tokens_per_wg - 1) / tokens_per_wg;
      local += nb[j];
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
      const int s = SPT * tid + j;
      if (s <= p.num_seqs) s_cum[s] = excl;
      excl += nb[j];
    }
    __syncthreads();
  }
  // heavy blocks (late query tokens see the most keys) are started first: walk the block list backwards
  const int item = s_cum[p.num_seqs] - 1 - static_cast<int>(blockIdx.x);
  if (item < 0) return;
  int seq;
  {
    int lo = 0, hi = p.num_seqs;
    while (lo + 1 < hi) {
      const int mid = (lo + hi) >> 1;
      if (s_cum[mid] <= item) {
        lo = mid;
      } else {
        hi = mid;
      }
    }
    seq = lo;
  }
  const int q_begin = p.cu_seqlens_q[seq];
  const int n_new = p.cu_seqlens_q[seq + 1] - q_begin;
  const int ctx = p.context_lens != nullptr ? p.context_lens[seq] : 0;
  const int tok0 = (item - s_cum[seq]) * tokens_per_wg;       // first new token of this block
  const int tok_cnt = min(tokens_per_wg, n_new - tok0);

  // keys this block may see: [key_lo, key_hi]
  const int key_hi = ctx + tok0 + tok_cnt - 1;
  int key_lo = 0;
  if (p.window_left >= 0) key_lo = max(0, ctx + tok0 - p.window_left);
  const int tile_lo = key_lo / TK;
  const int tile_hi = key_hi / TK;

  // ---- this lane's query rows ---------------------------------------------------------------------------------
  // row R = wave * 32 + 16 * nq + lr  ->  token tok0 + (R >> group_shift), head R & (group_pad - 1)
  int q_pos[kRowTiles];       // absolute position of the row's query, or -1 for a padding row
  int64_t row_elem[kRowTiles];  // element offset of the row in q / out
  V8 qop[kRowTiles][NS];
  float qbias[kRowTiles];
  const bool q_is_operand_type = (KIND == KV_BF16 && p.q_dtype == ARENO_DT_BF16) ||
                                 (KIND != KV_BF16 && p.q_dtype == ARENO_DT_F16);
#pragma unroll
  for (int nq = 0; nq < kRowTiles; ++nq) {
    const int r = wave * kRowsPerWave + 16 * nq + lr;
    const int t = r >> p.group_shift;
    const int hh = r & (p.group_pad - 1);
    const bool live = t < tok_cnt && hh < p.group;
    q_pos[nq] = live ? ctx + tok0 + t : -1;
    row_elem[nq] = (static_cast<int64_t>(q_begin + tok0 + t) * p.q_heads + kvh * p.group + hh) * D;
    float qsum = 0.0f;
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      uint4_t w = {0u, 0u, 0u, 0u};
      if (live) w = load16(p.q, (row_elem[nq] + (D / 4) * lk + 8 * sl) * 2);
      if (!q_is_operand_type) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
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
      qop[nq][sl] = __builtin_bit_cast(V8, w);
    }
    qbias[nq] = 0.0f;
    if constexpr (KIND == KV_I8) {
      qsum += wave_xor(qsum, 16);
      qsum += wave_xor(qsum, 32);
      qbias[nq] = kI8Offset * qsum;
    }
  }

  float4_t acc[kRowTiles][NB];
  float m_run[kRowTiles], l_run[kRowTiles], p_sum[kRowTiles];
#pragma unroll
  for (int nq = 0; nq < kRowTiles; ++nq) {
    m_run[nq] = kNegInf;
    l_run[nq] = 0.0f;
    p_sum[nq] = 0.0f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nq][nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  }

  // ---- cooperative tile fetch: thread tid owns chunks tid + 256 * i --------------------------------------------
  const int32_t* table_row = p.block_table + static_cast<int64_t>(seq) * p.max_blocks;
  constexpr int64_t row_bytes = static_cast<int64_t>(D) * ES;
  int ids[NLD];
  uint4_t kreg[NLD], vreg[NLD];
  scale_raw_t ksreg[NLD], vsreg[NLD];
  auto chunk_live = [&](int i) { return tid + kPrefillThreads * i < CHUNKS; };
  auto chunk_token = [&](int i) { return min(tid + kPrefillThreads * i, CHUNKS - 1) / LPT; };
  auto chunk_col = [&](int i) { return min(tid + kPrefillThreads * i, CHUNKS - 1) % LPT; };
  const bool packed = p.block_table == nullptr;  // K/V are (tokens, kv_heads, D): key t of the sequence is row q_begin + t
  auto issue_id_loads = [&](int tile) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int t = min(tile * TK + chunk_token(i), key_hi);
      ids[i] = packed ? 0 : table_row[p.bs_shift >= 0 ? (t >> p.bs_shift) : (t / p.block_size)];
    }
  };
  auto issue_kv_loads = [&](int tile) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int t = min(tile * TK + chunk_token(i), key_hi);
      const int slot = p.bs_shift >= 0 ? (t & (p.block_size - 1)) : (t % p.block_size);
      const int64_t row = packed ? (static_cast<int64_t>(q_begin) + t) * p.kv_heads + kvh
                                 : (static_cast<int64_t>(ids[i]) * p.block_size + slot) * p.kv_heads + kvh;
      kreg[i] = load16(p.k_cache, row * row_bytes + chunk_col(i) * 16);
      vreg[i] = load16(p.v_cache, row * row_bytes + chunk_col(i) * 16);
      if constexpr (T::kQuant) {
        ksreg[i] = static_cast<const scale_raw_t*>(p.k_scale)[row];
        vsreg[i] = static_cast<const scale_raw_t*>(p.v_scale)[row];
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

  issue_id_loads(tile_lo);
  issue_kv_loads(tile_lo);
  if (tile_lo < tile_hi) issue_id_loads(tile_lo + 1);

  for (int tile = tile_lo; tile <= tile_hi; ++tile) {
    const int k0 = tile * TK;
    // -- publish the fetched tile ------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int t = chunk_token(i);
      uint4_t kk = kreg[i], vv = vreg[i];
      if constexpr (KIND == KV_I8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          kk[j] ^= kI8Flip;
          vv[j] ^= kI8Flip;
        }
      }
      if (!chunk_live(i)) continue;
      *reinterpret_cast<uint4_t*>(s_k + t * RSK + chunk_col(i) * 16) = kk;
      *reinterpret_cast<uint4_t*>(s_v + v_row_of(t) * RSV + chunk_col(i) * 16) = vv;
      if (chunk_col(i) == 0) {
        if constexpr (T::kQuant) {
          s_ksc[t] = scale_value(ksreg[i]) * p.scale_log2e;
          s_vsc[t] = scale_value(vsreg[i]) * kPScale;
        } else {
          s_ksc[t] = p.scale_log2e;
          s_vsc[t] = kPScale;
        }
      }
    }
    __syncthreads();
    if (tile < tile_hi) {
      issue_kv_loads(tile + 1);
      if (tile + 1 < tile_hi) issue_id_loads(tile + 2);
    }

    // a wave whose rows all sit before this tile's first key has nothing to do here (causal); it still takes
    // part in the barriers
    const int wave_qmax = ctx + tok0 + min(tok_cnt, (((wave + 1) * kRowsPerWave - 1) >> p.group_shift) + 1) - 1;
    if (k0 <= wave_qmax && wave * kRowsPerWave < (tok_cnt << p.group_shift)) {
      // -- S^T = K . Q^T ------------------------------------------------------------------------------------------
      float s[kRowTiles][2][4];
#pragma unroll
      for (int tg = 0; tg < 2; ++tg) {
        const char* krow = s_k + (16 * tg + lr) * RSK + (D / 4) * ES * lk;
        uint32_t kw[NS * WPL];
#pragma unroll
        for (int q4 = 0; q4 < NS * WPL / 4; ++q4) {
          const uint4_t r = *reinterpret_cast<const uint4_t*>(krow + 16 * q4);
          kw[4 * q4 + 0] = r[0];
          kw[4 * q4 + 1] = r[1];
          kw[4 * q4 + 2] = r[2];
          kw[4 * q4 + 3] = r[3];
        }
        V8 kop[NS];
#pragma unroll
        for (int sl = 0; sl < NS; ++sl) kop[sl] = to_operand<KIND>(&kw[sl * WPL]);
        const float4_t sc = *reinterpret_cast<const float4_t*>(s_ksc + 16 * tg + 4 * lk);
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) {
          float4_t c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int sl = 0; sl < NS; ++sl) c = Ops::mfma(kop[sl], qop[nq][sl], c);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int kpos = k0 + 16 * tg + 4 * lk + j;
            bool ok = kpos <= q_pos[nq];
            if (p.window_left >= 0) ok = ok && kpos >= q_pos[nq] - p.window_left;
            s[nq][tg][j] = ok ? (c[j] - qbias[nq]) * sc[j] : kNegInf;
          }
        }
      }

      // -- online softmax per row ----------------------------------------------------------------------------------
      V8 pop[kRowTiles];
      const float4_t vs0 = *reinterpret_cast<const float4_t*>(s_vsc + 4 * lk);
      const float4_t vs1 = *reinterpret_cast<const float4_t*>(s_vsc + 16 + 4 * lk);
#pragma unroll
      for (int nq = 0; nq < kRowTiles; ++nq) {
        float mt = fmaxf(fmaxf(fmaxf(s[nq][0][0], s[nq][0][1]), fmaxf(s[nq][0][2], s[nq][0][3])),
                         fmaxf(fmaxf(s[nq][1][0], s[nq][1][1]), fmaxf(s[nq][1][2], s[nq][1][3])));
        mt = fmaxf(mt, wave_xor(mt, 16));
        mt = fmaxf(mt, wave_xor(mt, 32));
        const float m_new = fmaxf(m_run[nq], mt);
        const float m_safe = m_new == kNegInf ? 0.0f : m_new;
        const float alpha = fast_exp2(m_run[nq] - m_safe);
        m_run[nq] = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
          l_run[nq] *= alpha;
          p_sum[nq] *= alpha;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[nq][nb][j] *= alpha;
          }
        }
        float pe[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float e0 = fast_exp2(s[nq][0][j] - m_safe);
          const float e1 = fast_exp2(s[nq][1][j] - m_safe);
          l_run[nq] += e0 + e1;
          pe[j] = e0 * vs0[j];
          pe[4 + j] = e1 * vs1[j];
        }
        uint32_t pw[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          pw[j] = pack_pair<KIND>(pe[2 * j], pe[2 * j + 1]);
          if constexpr (KIND == KV_I8) {
            const Pair pr = __builtin_bit_cast(Pair, pw[j]);
            p_sum[nq] += static_cast<float>(pr.x) + static_cast<float>(pr.y);
          }
        }
        pop[nq] = __builtin_bit_cast(V8, uint4_t{pw[0], pw[1], pw[2], pw[3]});
      }

      // -- O^T += V^T . P^T -----------------------------------------------------------------------------------------
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        uint32_t vw[4];
        if constexpr (ES == 1) {
          const int r8 = lr >> 1;
          const int tok = r8 < 4 ? 4 * lk + r8 : 16 + 4 * lk + (r8 - 4);
          char* a = s_v + v_row_of(tok) * RSV + 16 * nb + 8 * (lr & 1);
          const int2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_int2*)a);
          vw[0] = static_cast<uint32_t>(r[0]);
          vw[1] = static_cast<uint32_t>(r[1]);
        } else {
          const int r4 = lr >> 2;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int tok = 16 * half + 4 * lk + r4;
            char* a = s_v + v_row_of(tok) * RSV + (16 * nb + 4 * (lr & 3)) * 2;
            const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
            const uint2_t u = __builtin_bit_cast(uint2_t, r);
            vw[2 * half] = u[0];
            vw[2 * half + 1] = u[1];
          }
        }
        const V8 vop = to_operand<KIND>(vw);
#pragma unroll
        for (int nq = 0; nq < kRowTiles; ++nq) acc[nq][nb] = Ops::mfma(vop, pop[nq], acc[nq][nb]);
      }
    }
    __syncthreads();  // every wave is done with the tile before the next one overwrites it
  }

  // ---- normalise and store ------------------------------------------------------------------------------------------
#pragma unroll
  for (int nq = 0; nq < kRowTiles; ++nq) {
    float l_tot = l_run[nq];
    l_tot += wave_xor(l_tot, 16);
    l_tot += wave_xor(l_tot, 32);
    float off = 0.0f;
    if constexpr (KIND == KV_I8) {
      float ps = p_sum[nq];
      ps += wave_xor(ps, 16);
      ps += wave_xor(ps, 32);
      off = kI8Offset * ps;
    }
    if (q_pos[nq] >= 0) {
      const float inv = 1.0f / (l_tot * kPScale);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int64_t e0 = row_elem[nq] + 16 * nb + 4 * lk;
        uint32_t lo, hi;
        const float o0 = (acc[nq][nb][0] - off) * inv, o1 = (acc[nq][nb][1] - off) * inv;
        const float o2 = (acc[nq][nb][2] - off) * inv, o3 = (acc[nq][nb][3] - off) * inv;
        if (p.q_dtype == ARENO_DT_BF16) {
          lo = float_to_bf16_bits(o0) | (float_to_bf16_bits(o1) << 16);
          hi = float_to_bf16_bits(o2) | (float_to_bf16_bits(o3) << 16);
        } else {
          lo = float_to_f16_bits(o0) | (float_to_f16_bits(o1) << 16);
          hi = float_to_f16_bits(o2) | (float_to_f16_bits(o3) << 16);
        }
        *reinterpret_cast<uint2_t*>(static_cast<char*>(p.out) + e0 * 2) = uint2_t{lo, hi};
      }
    }
  }
}

typedef void (*prefill_fn)(PrefillParams);

template <int KIND>
prefill_fn prefill_lookup(int head_dim, bool scale16) {
  if constexpr (KVTraits<KIND>::kQuant) {
    if (head_dim == 128) return scale16 ? prefill_mfma_kernel<KIND, 128, true> : prefill_mfma_kernel<KIND, 128, false>;
    if (head_dim == 64) return scale16 ? prefill_mfma_kernel<KIND, 64, true> : prefill_mfma_kernel<KIND, 64, false>;
  } else {
    if (head_dim == 128) return prefill_mfma_kernel<KIND, 128, false>;
    if (head_dim == 64) return prefill_mfma_kernel<KIND, 64, false>;
  }
  return nullptr;
}

int log2_exact_i(int x) {
  if (x <= 0 || (x & (x - 1)) != 0) return -1;
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}

}  // namespace

// block_table == nullptr selects packed K/V: cache->k / cache->v then point at (tokens, kv_heads, D) tensors and
// context_lens may be nullptr (no cached context).
int launch_prefill_mfma(const areno_paged_cache* cache, const void* q, void* out, int32_t q_dtype, int64_t tokens,
                        int32_t q_heads, int32_t num_seqs, const int32_t* block_table, int32_t max_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* context_lens, int32_t window_left,
                        float softmax_scale, void* stream) {
  const char* op = "areno_hip_paged_varlen_prefill";
  const int group = q_heads / cache->kv_heads;
  if (q_dtype != ARENO_DT_F16 && q_dtype != ARENO_DT_BF16) return ARENO_ERR_UNSUPPORTED;
  if (group > 16 || num_seqs > kMaxPrefillSeqs || tokens > 0x3fffffff) return ARENO_ERR_UNSUPPORTED;
  if (cache->kv_heads > 65535) return ARENO_ERR_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(cache->k) % 16 != 0 || reinterpret_cast<uintptr_t>(cache->v) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(q) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 8 != 0)
    return ARENO_ERR_UNSUPPORTED;
  const bool scale16 = cache->scale_dtype == ARENO_DT_F16;
  prefill_fn fn = nullptr;
  switch (cache->cache_dtype) {
    case ARENO_DT_BF16: fn = prefill_lookup<KV_BF16>(cache->head_dim, scale16); break;
    case ARENO_DT_F16: fn = prefill_lookup<KV_F16>(cache->head_dim, scale16); break;
    case ARENO_DT_I8: fn = prefill_lookup<KV_I8>(cache->head_dim, scale16); break;
    case ARENO_DT_FP8_E4M3: fn = prefill_lookup<KV_FP8>(cache->head_dim, scale16); break;
    default: break;
  }
  if (fn == nullptr) return ARENO_ERR_UNSUPPORTED;

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
  p.group = group;
  p.group_pad = 1;
  while (p.group_pad < group) p.group_pad <<= 1;
  p.group_shift = log2_exact_i(p.group_pad);
  p.block_size = cache->block_size;
  p.bs_shift = log2_exact_i(cache->block_size);
  p.max_blocks = max_blocks;
  p.window_left = window_left;
  p.q_dtype = q_dtype;
  p.scale_log2e = softmax_scale * kLog2e;
  // upper bound of query blocks without knowing the sequence lengths on the host
  const int tokens_per_wg = kRowsPerWg / p.group_pad;
  const int64_t max_blocks_q = (tokens + tokens_per_wg - 1) / tokens_per_wg + num_seqs;
  if (max_blocks_q > 0x7fffffff) return ARENO_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(fn, dim3(static_cast<unsigned>(max_blocks_q), cache->kv_heads), dim3(kPrefillThreads), 0,
                     static_cast<hipStream_t>(stream), p);
  return check_launch(op);
}

}  // namespace areno
