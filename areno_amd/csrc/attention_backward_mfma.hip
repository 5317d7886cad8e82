// Backward of the causal varlen / dense attention ops on the matrix cores (gfx950): 16-bit inputs, head dims 64 and
// 128.  Same contract as the vector-ALU kernels of attention_backward.hip (fp32 dQ, dK, dV from dO, Q, K, V and the
// saved output; areno/accel/csrc/attention.cu:244-524 in the reference), same two launches, no atomics:
//
//   dq kernel    a workgroup owns 64 or 128 packed query rows of one q head (four waves of 16 or 32 rows) and streams
//                the keys its rows may see in tiles of 32 through LDS.  Per tile, with the keys as the rows of the products (the
//                layout of the forward kernel):  S^T = K . Q^T  and  dP^T = V . dO^T  (two products per 16 keys and 32
//                elements of the head), the online softmax of the forward on S^T, dS^T = P^T * (dP^T - dO . O), and
//                dQ^T += K^T . dS^T  with the lane's own dS^T values as the B operand and K^T read transposed from the
//                same LDS tile.  A row's softmax reference moves as in the forward (the accumulator is rescaled), so
//                one pass over the keys gives dQ, the row's log-sum-exp and dO . O (left in the workspace).
//   dkv kernel   a workgroup owns 64 or 32 packed key rows of one kv head (16 per wave) and streams, for every q head
//                of the group, the query rows that may see them in tiles of 32 (Q and dO tiles in LDS, the rows'
//                statistics next to them):  S = Q . K^T,  dP = dO . V^T,  P = exp2(S - lse),  dS = P * (dP - dO . O),
//                dV^T += dO^T . P  and  dK^T += Q^T . dS.  Every gradient element has one owner; in a small launch
//                the stream of tiles is split over two or four sets of waves whose sums are added in a fixed order.
// Both launches take their blocks in an order (or in pairs) that lets their workgroups end together: see
// block_in_cost_order and the dkv kernel.
//
// The streamed index of a tile (keys in the dq kernel, queries in the dkv kernel) is the contraction index of the
// second pair of products; a 16 x 16 product leaves element 4 g + j of that index in lane group g, which is exactly
// how the next product wants its B operand, and the A operand comes from the LDS tile through transposing reads
// (ds_read_b64_tr_b16), so nothing is shuffled between the products.
// Geometry as in attention_backward.hip: sequence s has queries [cu_q[s], cu_q[s+1]) at positions ctx[s] + i and keys
// [cu_k[s], cu_k[s+1]) at positions 0 ..; a query at position t sees keys max(0, t - window) .. t.  A block of
// packed rows may hold rows of several sequences; it goes through them one after the other, the rows of the others
// masked.

#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <type_traits>

#include "attention_backward.hpp"
#include "backward_order.hpp"
#include "decode_mfma_kernels.hpp"

namespace areno {
namespace {

constexpr int kBmWaves = 4;
constexpr int kBmThreads = kBmWaves * kWave;
constexpr int kBmRows = 16 * kBmWaves;  // packed rows a workgroup owns
constexpr int kBmTile = 32;             // streamed rows per step
constexpr float kBmNegInf = -__builtin_huge_valf();

// the last sequence that starts at or in front of `row` (the one that holds it, when the row exists)
__device__ __forceinline__ int seq_of_row(const int32_t* cu, int num_seqs, int64_t row) {
  int lo = 0, hi = num_seqs;
  while (lo + 1 < hi) {
    const int mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(cu[mid]) <= row) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

// A tile of 32 rows x D 16-bit elements in LDS, row stride D * 2 + 16 bytes: the row operands (16 lanes read the same
// 16-byte chunk of 16 rows) meet every bank once, the transposed ones (32 lanes read 32 bytes of 8 consecutive rows)
// meet every bank twice.  (A layout without any bank conflict -- rows back to back, the chunks of a row permuted by
// a function of the row -- was measured, with four and with eight waves on a compute unit's LDS: LDS is busy 40 %
// less with it and no launch got faster, small ones 3-8 % slower from the address registers it takes.)  Staging: every thread moves kChunks 16-byte chunks of a tensor
// through registers.
template <int D>
struct BmTile {
  static constexpr int RS = D * 2 + 16;
  static constexpr int kChunksPerRow = D * 2 / 16;
  static constexpr int kChunks = kBmTile * kChunksPerRow / kBmThreads;  // per thread: 1 (D = 64) or 2 (D = 128)
  static_assert(kBmTile * kChunksPerRow % kBmThreads == 0, "tile chunks");
  static __device__ __forceinline__ int chunk_pos(int r, int c) { return r * RS + (c << 4); }
};

// Operand reads.  Row operand (A of the first pair of products): row 16 tg + lr of the tile, elements
// (D / 4) lk + 8 sl .. + 8 -- the same split of the head over the four lane groups as the register operands.
template <int KIND, typename T, int D>
__device__ __forceinline__ typename MfmaOps<KIND>::vec8 tile_row_operand(const char* tile, int tg, int sl, int lr, int lk) {
  using V8 = typename MfmaOps<KIND>::vec8;
  return *reinterpret_cast<const V8*>(tile + T::chunk_pos(16 * tg + lr, (D / 32) * lk + sl));
}
// Transposed operand (A of the second pair): head elements 16 nb + lr as rows, the tile's 32 rows as the contraction
// index in the order lane group lk holds them after the first pair (rows 4 lk .. 4 lk + 3, then 16 + 4 lk .. + 3).
template <int KIND, typename T>
__device__ __forceinline__ typename MfmaOps<KIND>::vec8 tile_transposed_operand(char* tile, int nb, int lr, int lk) {
  using V8 = typename MfmaOps<KIND>::vec8;
  uint32_t w[4];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int row = 16 * half + 4 * lk + (lr >> 2);
    char* a = tile + T::chunk_pos(row, 2 * nb + ((lr & 3) >> 1)) + 8 * (lr & 1);
    const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)a);
    const uint2_t u = __builtin_bit_cast(uint2_t, r);
    w[2 * half] = u[0];
    w[2 * half + 1] = u[1];
  }
  return __builtin_bit_cast(V8, uint4_t{w[0], w[1], w[2], w[3]});
}
// eight values of the streamed index, as a lane holds them after the first pair of products ([tg][j]), as B operand
template <int KIND>
__device__ __forceinline__ typename MfmaOps<KIND>::vec8 streamed_operand(const float (&x)[2][4]) {
  using V8 = typename MfmaOps<KIND>::vec8;
  return __builtin_bit_cast(V8, uint4_t{pack_pair<KIND>(x[0][0], x[0][1]), pack_pair<KIND>(x[0][2], x[0][3]),
                                        pack_pair<KIND>(x[1][0], x[1][1]), pack_pair<KIND>(x[1][2], x[1][3])});
}
template <int KIND>
__device__ __forceinline__ float operand_element(uint32_t word, int hi) {
  const uint32_t bits = hi ? word >> 16 : word & 0xffffu;
  return KIND == KV_BF16 ? bf16_bits_to_float(bits) : f16_bits_to_float(bits);
}

// ---- dQ (and the rows' statistics) ------------------------------------------------------------------------------------
// CB = blocks of 16 query rows a wave owns: 1 (a workgroup of four waves owns 64 packed rows) or 2 (128 rows).  With
// two, every operand read from the LDS tile serves two products (the tile's K and V rows in the first pair, K^T in
// the second), at twice the registers for the rows' operands and sums.
template <int KIND, int D, int CB>
__global__ __launch_bounds__(kBmThreads, 2) void bwd_mfma_dq_kernel(BwdParams p) {
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using T = BmTile<D>;
  constexpr int NS = D / 32, NB = D / 16;
  constexpr int kRows = kBmRows * CB;  // packed rows of the workgroup
  constexpr int kWaveRows = 16 * CB;
  __shared__ __attribute__((aligned(16))) char s_k[kBmTile * T::RS];
  __shared__ __attribute__((aligned(16))) char s_v[kBmTile * T::RS];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = uniform(tid >> 6);  // (in a scalar register: what follows from it is scalar work and scalar branches)
  const int lr = lane & 15, lk = lane >> 4;
  // workgroups in launch order: the heads of a block next to each other, the blocks by cost
  const int h = static_cast<int>(blockIdx.x % static_cast<unsigned>(p.q_heads));
  const int kvh = h / (p.q_heads / p.kv_heads);
  const int64_t q_blocks = (p.q_tokens + kRows - 1) / kRows;
  const int64_t r0 = block_in_cost_order(blockIdx.x / static_cast<unsigned>(p.q_heads), q_blocks, p.num_seqs, true) * kRows;
  const int64_t block_end = r0 + kRows < p.q_tokens ? r0 + kRows : p.q_tokens;
  const int64_t wave_row0 = r0 + kWaveRows * wave;
  int64_t row[CB];  // this lane's query rows (columns of the products)
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) row[cb] = wave_row0 + 16 * cb + lr;

  for (int s = seq_of_row(p.cu_q, p.num_seqs, r0); s < p.num_seqs; ++s) {
    const int64_t sq0 = p.cu_q[s], sq1 = p.cu_q[s + 1];
    if (sq0 >= block_end) break;
    const int64_t q_lo = sq0 > r0 ? sq0 : r0, q_hi = sq1 < block_end ? sq1 : block_end;
    if (q_lo >= q_hi) continue;
    const int ctx = p.ctx != nullptr ? p.ctx[s] : 0;
    const int64_t k_base = p.cu_k[s];
    const int n_k = p.cu_k[s + 1] - p.cu_k[s];
    bool live[CB];
    int pos[CB];
    bool wave_live = false, wave_full = true;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      live[cb] = row[cb] >= q_lo && row[cb] < q_hi;
      pos[cb] = live[cb] ? ctx + static_cast<int>(row[cb] - sq0) : -1;
      const uint64_t live_lanes = __builtin_amdgcn_ballot_w64(live[cb]);
      wave_live = wave_live || live_lanes != 0;
      wave_full = wave_full && live_lanes == ~0ull;
    }
    // (the positions of the wave's query rows, when all of them belong to this sequence)
    const int wave_pos_lo = ctx + static_cast<int>(wave_row0 - sq0), wave_pos_hi = wave_pos_lo + kWaveRows - 1;
    const int pos_min = ctx + static_cast<int>(q_lo - sq0), pos_max = ctx + static_cast<int>(q_hi - 1 - sq0);
    const int key_lo = p.window_left >= 0 ? (pos_min - p.window_left > 0 ? pos_min - p.window_left : 0) : 0;
    const int key_hi = pos_max < n_k - 1 ? pos_max : n_k - 1;

    // this lane's parts of its rows of Q and dO (B operands), and dO . O
    int64_t row_elem[CB];
    V8 qop[CB][NS], gop[CB][NS];
    float delta[CB];
    float4_t acc[CB][NB];
    float m_run[CB], l_lane[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      row_elem[cb] = (row[cb] * p.q_heads + h) * D;
      float d = 0.0f;
#pragma unroll
      for (int sl = 0; sl < NS; ++sl) {
        uint4_t qw = {0u, 0u, 0u, 0u}, gw = qw, ow = qw;
        if (live[cb]) {
          const int64_t off = (row_elem[cb] + (D / 4) * lk + 8 * sl) * 2;
          qw = load16(p.q, off);
          gw = load16(p.grad_out, off);
          ow = load16(p.out, off);
        }
        qop[cb][sl] = __builtin_bit_cast(V8, qw);
        gop[cb][sl] = __builtin_bit_cast(V8, gw);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          d += operand_element<KIND>(gw[j], 0) * operand_element<KIND>(ow[j], 0) +
               operand_element<KIND>(gw[j], 1) * operand_element<KIND>(ow[j], 1);
        }
      }
      delta[cb] = rows_sum(d);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[cb][nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
      m_run[cb] = kBmNegInf;
      l_lane[cb] = 0.0f;
    }

    if (key_hi >= key_lo) {  // (the same for the whole workgroup)
      const int t0 = key_lo / kBmTile, t1 = key_hi / kBmTile;
      uint4_t kreg[T::kChunks], vreg[T::kChunks];
      auto fetch = [&](int t) {
#pragma unroll
        for (int i = 0; i < T::kChunks; ++i) {
          const int c = tid + kBmThreads * i;
          const int r = c / T::kChunksPerRow, col = c % T::kChunksPerRow;
          const int key = kBmTile * t + r < n_k ? kBmTile * t + r : n_k - 1;  // rows past the end repeat the last key
          const int64_t off = ((k_base + key) * p.kv_heads + kvh) * (D * 2) + col * 16;
          kreg[i] = load16(p.k, off);
          vreg[i] = load16(p.v, off);
        }
      };
      auto publish = [&]() {
#pragma unroll
        for (int i = 0; i < T::kChunks; ++i) {
          const int c = tid + kBmThreads * i;
          const int r = c / T::kChunksPerRow, col = c % T::kChunksPerRow;
          *reinterpret_cast<uint4_t*>(s_k + T::chunk_pos(r, col)) = kreg[i];
          *reinterpret_cast<uint4_t*>(s_v + T::chunk_pos(r, col)) = vreg[i];
        }
      };
      fetch(t0);
      __syncthreads();  // the tiles' previous readers (an earlier sequence of this block) are done
      publish();
      __syncthreads();
      for (int t = t0; t <= t1; ++t) {
        if (t < t1) fetch(t + 1);
        if (wave_live) {
          float sc[CB][2][4], dp[CB][2][4];
          auto first_products = [&](auto masked) {
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
              float4_t c1[CB], c2[CB];
#pragma unroll
              for (int cb = 0; cb < CB; ++cb) c1[cb] = c2[cb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
              for (int sl = 0; sl < NS; ++sl) {
                const V8 k_rows = tile_row_operand<KIND, T, D>(s_k, tg, sl, lr, lk);
                const V8 v_rows = tile_row_operand<KIND, T, D>(s_v, tg, sl, lr, lk);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                  c1[cb] = Ops::mfma(k_rows, qop[cb][sl], c1[cb]);
                  c2[cb] = Ops::mfma(v_rows, gop[cb][sl], c2[cb]);
                }
              }
#pragma unroll
              for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  sc[cb][tg][j] = c1[cb][j];  // (the softmax scale goes in with the reference, below)
                  if constexpr (decltype(masked)::value) {
                    const int key = kBmTile * t + 16 * tg + 4 * lk + j;
                    const bool ok =
                        key <= pos[cb] && key < n_k && (p.window_left < 0 || key >= pos[cb] - p.window_left);
                    sc[cb][tg][j] = ok ? sc[cb][tg][j] : kBmNegInf;
                  }
                  dp[cb][tg][j] = c2[cb][j];
                }
              }
            }
          };
          // most tiles lie below the diagonal and inside the window as a whole: every query row of this wave sees
          // every key of the tile, and nothing needs a mask
          const int key_first = kBmTile * t, key_last = key_first + kBmTile - 1;
          const bool plain = wave_full && key_last < n_k && key_last <= wave_pos_lo &&
                             (p.window_left < 0 || key_first >= wave_pos_hi - p.window_left);
          if (plain) {
            first_products(std::false_type{});
          } else {
            first_products(std::true_type{});
          }
          V8 dsop[CB];
          bool moved = false;
          float alpha[CB];
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            float mt = sc[cb][0][0];
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
              for (int j = 0; j < 4; ++j) mt = fmaxf(mt, sc[cb][tg][j]);
            }
            mt = rows_max(mt);
            const float m_new = fmaxf(m_run[cb], mt * p.scale_log2e);  // (the scale is positive)
            const float m_ref = m_new == kBmNegInf ? 0.0f : m_new;
            alpha[cb] = fast_exp2(m_run[cb] - m_ref);  // 0 while the row has seen no key
            m_run[cb] = m_new;
            float ds[2][4], psum = 0.0f;
#pragma unroll
            for (int tg = 0; tg < 2; ++tg) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                // (exp2(-inf) = 0: masked keys)
                const float pe = fast_exp2(__builtin_fmaf(sc[cb][tg][j], p.scale_log2e, -m_ref));
                psum += pe;
                ds[tg][j] = pe * (dp[cb][tg][j] - delta[cb]);
              }
            }
            l_lane[cb] = l_lane[cb] * alpha[cb] + psum;
            dsop[cb] = streamed_operand<KIND>(ds);
            moved = moved || __builtin_amdgcn_ballot_w64(alpha[cb] != 1.0f) != 0;
          }
          if (moved) {  // (after the first tiles a new maximum is rare)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
              for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[cb][nb][j] *= alpha[cb];
              }
            }
          }
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const V8 k_cols = tile_transposed_operand<KIND, T>(s_k, nb, lr, lk);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[cb][nb] = Ops::mfma(k_cols, dsop[cb], acc[cb][nb]);
          }
        }
        __syncthreads();  // every wave has read tile t
        if (t < t1) publish();
        __syncthreads();
      }
    }

    // dQ = scale / l * sum_k p_k (dP_k - dO . O) K_k; the row's log-sum-exp (log2 domain) and dO . O for the dkv kernel
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
      const float l_tot = rows_sum(l_lane[cb]);
      if (live[cb]) {
        const float f = l_tot > 0.0f ? p.scale / l_tot : 0.0f;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          store_grad4(p.grad_q, row_elem[cb] + 4 * lk + 16 * nb, acc[cb][nb][0] * f, acc[cb][nb][1] * f,
                      acc[cb][nb][2] * f, acc[cb][nb][3] * f, p.grad_dtype);
        }
        if (lk == 0) {
          float* st = p.row_stats + (row[cb] * p.q_heads + h) * 2;
          // a row without visible keys gets a reference no score reaches: its probabilities come out as zeros
          st[0] = l_tot > 0.0f ? m_run[cb] + __builtin_log2f(l_tot) : __builtin_huge_valf();
          st[1] = delta[cb];
        }
      }
    }
  }
}

// ---- dK, dV -------------------------------------------------------------------------------------------------------------
// A workgroup owns a block of KR packed key rows of one kv head, or two of them one after the other: block i and
// block blocks - 1 - i.  A key block early in its sequence is seen by all later queries and one late in it by few.
// A launch of many workgroups per compute unit evens that out by starting the expensive blocks first
// (block_in_cost_order); in a launch of about one workgroup per unit nothing comes after the expensive block to
// fill the gap, and there the pairs help: for sequences of about equal length the costs of such a pair add up to
// the same for every i, so the workgroups end together.  (The launcher says which by the size of the grid.)
// The workgroup has P parts of KR / 16 waves.  Every part owns all KR key rows (16 per wave) and takes every P-th
// step of the stream of query tiles (tiles and statistics of its own in LDS); the sums of parts 1 .. P - 1 go to
// part 0 through LDS at the end of a block, in a fixed order.  More parts shorten the chain of steps a block is:
// (KR, P) = (64, 1) four waves, two workgroups per compute unit, for launches that fill the units several times;
// (64, 2) and (32, 4) eight waves, for launches of about one workgroup per unit.
template <int D, int KR, int P>
struct DkvShape {
  static constexpr int kKeyWaves = KR / 16;
  static constexpr int kPartThreads = kKeyWaves * kWave;
  static constexpr int kThreads = kPartThreads * P;
  static constexpr int RS = BmTile<D>::RS;
  static constexpr int kChunksPerRow = BmTile<D>::kChunksPerRow;
  static constexpr int kChunks = kBmTile * kChunksPerRow / kPartThreads;  // 16-byte chunks of a tile per thread of a part
  static_assert(kBmTile * kChunksPerRow % kPartThreads == 0, "tile chunks");
  static constexpr int kTile = kBmTile * RS;
  static constexpr int kStat = kBmTile * 2 * 4;
  // per part and buffer: a Q tile, a dO tile, the rows' statistics
  static constexpr int kBuffer = 2 * kTile + kStat;
  static constexpr int kStream = P * 2 * kBuffer;
  static constexpr int kSums = (P - 1) * kPartThreads * (D / 16) * 2 * 16;  // a float4 per lane, block of 16 and tensor
  static constexpr int kLdsBytes = kStream > kSums ? kStream : kSums;
};
extern __shared__ __attribute__((aligned(16))) char bm_dkv_lds[];

template <int KIND, int D, int KR, int P>
__global__ __launch_bounds__((DkvShape<D, KR, P>::kThreads), (DkvShape<D, KR, P>::kThreads == 256 ? 2 : 1)) void bwd_mfma_dkv_kernel(
    BwdParams p) {
  using Ops = MfmaOps<KIND>;
  using V8 = typename Ops::vec8;
  using T = BmTile<D>;
  using L = DkvShape<D, KR, P>;
  constexpr int NS = D / 32, NB = D / 16;

  // (the same for a wave, and told so: the part's steps, cursors and loop counts then live in scalar registers)
  const int part = P > 1 ? uniform(static_cast<int>(threadIdx.x) / L::kPartThreads) : 0;
  const int tid = P > 1 ? static_cast<int>(threadIdx.x) % L::kPartThreads : static_cast<int>(threadIdx.x);  // in the part
  char* const lds = bm_dkv_lds + part * (2 * L::kBuffer);
  auto s_q = [&](int buf) { return lds + buf * L::kBuffer; };
  auto s_g = [&](int buf) { return lds + buf * L::kBuffer + L::kTile; };
  auto s_stat = [&](int buf) { return reinterpret_cast<float*>(lds + buf * L::kBuffer + 2 * L::kTile); };  // [row][2]

  const int lane = tid & (kWave - 1);
  const int wave = uniform(tid >> 6);
  const int lr = lane & 15, lk = lane >> 4;
  const int kvh = static_cast<int>(blockIdx.x % static_cast<unsigned>(p.kv_heads));
  const int group = p.q_heads / p.kv_heads;
  const int64_t k_blocks = (p.k_tokens + KR - 1) / KR;
  const int64_t wg = blockIdx.x / static_cast<unsigned>(p.kv_heads);
  // (launched with a workgroup per pair of blocks, or with one per block: then in cost order, one block each)
  const bool paired = gridDim.x / static_cast<unsigned>(p.kv_heads) < k_blocks;
  const int64_t first_block = paired ? wg : block_in_cost_order(wg, k_blocks, p.num_seqs, false);

  for (int half = 0; half < 2; ++half) {
    const int64_t block = half == 0 ? first_block : k_blocks - 1 - first_block;
    // (no second block without pairs, and none for the middle one of an odd number of blocks)
    if (half == 1 && (!paired || block <= first_block)) break;
    const int64_t r0 = block * KR;
    const int64_t block_end = r0 + KR < p.k_tokens ? r0 + KR : p.k_tokens;
    const int64_t row = r0 + 16 * wave + lr;  // this lane's key row (a column of the products)
    const bool row_exists = row < p.k_tokens;

    // this lane's parts of its row of K and V (B operands)
    const int64_t row_elem = (row * p.kv_heads + kvh) * D;
    V8 kop[NS], vop[NS];
#pragma unroll
    for (int sl = 0; sl < NS; ++sl) {
      uint4_t kw = {0u, 0u, 0u, 0u}, vw = kw;
      if (row_exists) {
        const int64_t off = (row_elem + (D / 4) * lk + 8 * sl) * 2;
        kw = load16(p.k, off);
        vw = load16(p.v, off);
      }
      kop[sl] = __builtin_bit_cast(V8, kw);
      vop[sl] = __builtin_bit_cast(V8, vw);
    }
    float4_t acc_k[NB], acc_v[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc_k[nb] = acc_v[nb] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

    for (int s = seq_of_row(p.cu_k, p.num_seqs, r0); s < p.num_seqs; ++s) {
      const int64_t sk0 = p.cu_k[s], sk1 = p.cu_k[s + 1];
      if (sk0 >= block_end) break;
      const int64_t k_lo = sk0 > r0 ? sk0 : r0, k_hi = sk1 < block_end ? sk1 : block_end;
      if (k_lo >= k_hi) continue;
      const int ctx = p.ctx != nullptr ? p.ctx[s] : 0;
      const int64_t q_base = p.cu_q[s];
      const int n_q = p.cu_q[s + 1] - p.cu_q[s];
      const bool live = row >= k_lo && row < k_hi;
      const int key = live ? static_cast<int>(row - sk0) : -1;  // this lane's key position in the sequence
      const uint64_t live_lanes = __builtin_amdgcn_ballot_w64(live);
      const bool wave_live = live_lanes != 0, wave_full = live_lanes == ~0ull;
      // (the wave's 16 key rows, when all of them belong to this sequence)
      const int wave_key_lo = static_cast<int>(r0 + 16 * wave - sk0), wave_key_hi = wave_key_lo + 15;
      // queries i (position ctx + i) that see one of the block's keys: key <= ctx + i <= key + window
      const int key_min = static_cast<int>(k_lo - sk0), key_max = static_cast<int>(k_hi - 1 - sk0);
      const int i_lo = key_min - ctx > 0 ? key_min - ctx : 0;
      int i_hi = n_q - 1;
      if (p.window_left >= 0 && key_max + p.window_left - ctx < i_hi) i_hi = key_max + p.window_left - ctx;
      if (i_hi < i_lo) continue;  // (the same for the whole workgroup)
      const int t0 = i_lo / kBmTile, t1 = i_hi / kBmTile;
      const int tiles = t1 - t0 + 1;
      // the stream: tiles of every q head of the group, head by head; this part takes steps part, part + P, ...
      const int stream_steps = tiles * group;
      const int steps = (stream_steps - part + P - 1) / P;  // this part's
      const int rounds = (stream_steps + P - 1) / P;        // the longest part's: every part keeps the barriers of all
      // (head, tile) of a step of the stream, counted up by P steps at a time
      struct Cursor {
        int head, tile;
      };
      auto advance = [&](Cursor& c) {
        c.tile += P;
        while (c.tile > t1) {
          c.tile -= tiles;
          ++c.head;
        }
      };
      Cursor first = {kvh * group, t0 + part};
      while (first.tile > t1) {
        first.tile -= tiles;
        ++first.head;
      }

      // Two register sets hold the tiles of the next two steps while they are in flight; a step computes on one of
      // the two LDS buffers, moves the next step's tile into the other one and asks for the tile two steps further on.
      struct Staged {
        uint4_t q[L::kChunks], g[L::kChunks];
        float2_t stat;
      };
      Staged set_a, set_b;
      Cursor fetch_at = first;
      int fetched = 0;
      auto fetch = [&](Staged& st) {
        if (fetched >= steps) return;
        ++fetched;
        const int hq = fetch_at.head, t = fetch_at.tile;
        advance(fetch_at);
#pragma unroll
        for (int i = 0; i < L::kChunks; ++i) {
          const int c = tid + L::kPartThreads * i;
          const int r = c / T::kChunksPerRow, col = c % T::kChunksPerRow;
          const int qi = kBmTile * t + r < n_q ? kBmTile * t + r : n_q - 1;  // rows past the end repeat the last query
          const int64_t off = ((q_base + qi) * p.q_heads + hq) * (D * 2) + col * 16;
          st.q[i] = load16(p.q, off);
          st.g[i] = load16(p.grad_out, off);
        }
        if (tid < kBmTile) {
          const int qi = kBmTile * t + tid < n_q ? kBmTile * t + tid : n_q - 1;
          st.stat = *reinterpret_cast<const float2_t*>(p.row_stats + ((q_base + qi) * p.q_heads + hq) * 2);
        }
      };
      auto publish = [&](const Staged& st, int buf) {
#pragma unroll
        for (int i = 0; i < L::kChunks; ++i) {
          const int c = tid + L::kPartThreads * i;
          const int r = c / T::kChunksPerRow, col = c % T::kChunksPerRow;
          *reinterpret_cast<uint4_t*>(s_q(buf) + T::chunk_pos(r, col)) = st.q[i];
          *reinterpret_cast<uint4_t*>(s_g(buf) + T::chunk_pos(r, col)) = st.g[i];
        }
        if (tid < kBmTile) *reinterpret_cast<float2_t*>(s_stat(buf) + 2 * tid) = st.stat;
      };
      Cursor at = first;  // the step being computed
      // one step: the products of the tile in LDS buffer `buf`; between them the next step's tile goes from `next`
      // into the other buffer and `next` is asked to fetch again
      auto step_on = [&](int step, int buf, Staged& next) {
        const int t = at.tile;
        advance(at);
        const bool compute = wave_live && step < steps;
        float pr[2][4], ds[2][4];
        auto first_products = [&](auto masked) {
#pragma unroll
          for (int tg = 0; tg < 2; ++tg) {
            // the statistics of the four query rows this lane gets from the products: rows 16 tg + 4 lk .. + 3
            const float4_t st01 = *reinterpret_cast<const float4_t*>(s_stat(buf) + 2 * (16 * tg + 4 * lk));
            const float4_t st23 = *reinterpret_cast<const float4_t*>(s_stat(buf) + 2 * (16 * tg + 4 * lk + 2));
            const float lse[4] = {st01[0], st01[2], st23[0], st23[2]};
            const float dlt[4] = {st01[1], st01[3], st23[1], st23[3]};
            float4_t c1 = {0.0f, 0.0f, 0.0f, 0.0f}, c2 = c1;
#pragma unroll
            for (int sl = 0; sl < NS; ++sl) {
              c1 = Ops::mfma(tile_row_operand<KIND, T, D>(s_q(buf), tg, sl, lr, lk), kop[sl], c1);
              c2 = Ops::mfma(tile_row_operand<KIND, T, D>(s_g(buf), tg, sl, lr, lk), vop[sl], c2);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float x = c1[j] * p.scale_log2e - lse[j];
              if constexpr (decltype(masked)::value) {
                const int qi = kBmTile * t + 16 * tg + 4 * lk + j;  // query of the sequence
                const int pos = ctx + qi;
                const bool ok = live && qi < n_q && key <= pos && (p.window_left < 0 || key >= pos - p.window_left);
                x = ok ? x : kBmNegInf;
              }
              // (a query without visible keys has +inf as its log-sum-exp: exp2(-inf) = 0 either way)
              const float pe = fast_exp2(x);
              pr[tg][j] = pe;
              ds[tg][j] = pe * (c2[j] - dlt[j]);
            }
          }
        };
        if (compute) {
          // most tiles lie below the diagonal and inside the window as a whole: every query of the tile sees every
          // key of this wave, and nothing needs a mask
          const int pos_lo = ctx + kBmTile * t, pos_hi = pos_lo + kBmTile - 1;
          const bool plain = wave_full && kBmTile * t + kBmTile <= n_q && pos_lo >= wave_key_hi &&
                             (p.window_left < 0 || pos_hi - p.window_left <= wave_key_lo);
          if (plain) {
            first_products(std::false_type{});
          } else {
            first_products(std::true_type{});
          }
        }
        if (step + 1 < steps) publish(next, buf ^ 1);
        fetch(next);
        if (compute) {
          const V8 pop = streamed_operand<KIND>(pr);
          const V8 dsop = streamed_operand<KIND>(ds);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            acc_v[nb] = Ops::mfma(tile_transposed_operand<KIND, T>(s_g(buf), nb, lr, lk), pop, acc_v[nb]);
            acc_k[nb] = Ops::mfma(tile_transposed_operand<KIND, T>(s_q(buf), nb, lr, lk), dsop, acc_k[nb]);
          }
        }
        __syncthreads();  // every wave has read this step's tile, the next one is in place
      };
      // (every wave has passed a barrier behind the last use of the buffers: an earlier sequence's last step, or the
      // hand-over of the block before)
      fetch(set_a);
      fetch(set_b);
      if (steps > 0) publish(set_a, 0);
      fetch(set_a);
      __syncthreads();
      for (int step = 0; step < rounds; step += 2) {
        step_on(step, 0, set_b);
        if (step + 1 < rounds) step_on(step + 1, 1, set_a);
      }
    }

    if constexpr (P > 1) {
      // the other parts' sums to part 0: a float4 per lane, block of 16 and tensor, lanes next to each other
      // (the tiles' last readers have passed a barrier, or no step ran at all)
      float4_t* sums = reinterpret_cast<float4_t*>(bm_dkv_lds);
      if (part > 0) {
        float4_t* mine = sums + (part - 1) * (2 * NB * L::kPartThreads);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          mine[(2 * nb) * L::kPartThreads + tid] = acc_k[nb];
          mine[(2 * nb + 1) * L::kPartThreads + tid] = acc_v[nb];
        }
      }
      __syncthreads();
      if (part == 0) {
#pragma unroll
        for (int other = 1; other < P; ++other) {
          const float4_t* theirs = sums + (other - 1) * (2 * NB * L::kPartThreads);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const float4_t dk = theirs[(2 * nb) * L::kPartThreads + tid], dv = theirs[(2 * nb + 1) * L::kPartThreads + tid];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              acc_k[nb][j] += dk[j];
              acc_v[nb][j] += dv[j];
            }
          }
        }
      }
      __syncthreads();  // the sums are read: the second block's tiles may overwrite them
    }

    // every gradient element is written, also the zeros of keys no query sees
    if (part == 0 && row_exists) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int64_t at_elem = row_elem + 4 * lk + 16 * nb;
        store_grad4(p.grad_k, at_elem, acc_k[nb][0] * p.scale, acc_k[nb][1] * p.scale, acc_k[nb][2] * p.scale,
                    acc_k[nb][3] * p.scale, p.grad_dtype);
        store_grad4(p.grad_v, at_elem, acc_v[nb][0], acc_v[nb][1], acc_v[nb][2], acc_v[nb][3], p.grad_dtype);
      }
    }
  }
}

typedef void (*bm_fn)(BwdParams);
constexpr int64_t kBmComputeUnits = 256;

// the dkv kernel of a (type, head dim, key rows per block, parts) with its launch shape; more than 64 KB of LDS has
// to be allowed once per device
struct DkvLaunch {
  bm_fn fn;
  int lds_bytes, threads, key_rows;
};
template <int KIND, int D, int KR, int P>
DkvLaunch dkv_launch() {
  using L = DkvShape<D, KR, P>;
  const bm_fn fn = bwd_mfma_dkv_kernel<KIND, D, KR, P>;
  if constexpr (L::kLdsBytes > 64 * 1024) {
    static std::atomic<uint64_t> allowed_on{0};  // one bit per device (the attribute belongs to the device's copy)
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return DkvLaunch{nullptr, 0, 0, 0};
    if ((allowed_on.load(std::memory_order_acquire) >> device & 1) == 0) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                              L::kLdsBytes) != hipSuccess) {
        (void)hipGetLastError();
        return DkvLaunch{nullptr, 0, 0, 0};
      }
      allowed_on.fetch_or(uint64_t{1} << device, std::memory_order_release);
    }
  }
  return DkvLaunch{fn, L::kLdsBytes, L::kThreads, KR};
}
template <int KIND, int D>
DkvLaunch dkv_launch(int parts) {
  if (parts == 4) return dkv_launch<KIND, D, 32, 4>();
  return parts == 2 ? dkv_launch<KIND, D, 64, 2>() : dkv_launch<KIND, D, 64, 1>();
}

}  // namespace

int launch_attention_backward_mfma(const BwdParams& p, void* stream) {
  if (p.dtype != ARENO_DT_BF16 && p.dtype != ARENO_DT_F16) return ARENO_ERR_UNSUPPORTED;
  if (p.head_dim != 64 && p.head_dim != 128) return ARENO_ERR_UNSUPPORTED;
  if (p.q_heads > 65535 || p.kv_heads > 65535) return ARENO_ERR_UNSUPPORTED;
  const int64_t q_blocks = (p.q_tokens + kBmRows - 1) / kBmRows, k_blocks = (p.k_tokens + kBmRows - 1) / kBmRows;
  if (q_blocks * p.q_heads > 0x7fffffffLL || k_blocks * p.kv_heads > 0x7fffffffLL) return ARENO_ERR_UNSUPPORTED;
  const bool bf16 = p.dtype == ARENO_DT_BF16;
  // The dkv kernel's shape by the size of the launch.  About one workgroup per compute unit: pairs of blocks of 32
  // key rows, eight waves in four parts (2 x 2 048 tokens, 28 / 4 heads: 527 -> 463 us for both launches; one
  // sequence of 4 096: 975 -> 814 us).  Up to 4 per unit at head dim 128 and 2 at head dim 64: a block of 64 rows
  // each, in cost order, eight waves in two parts (2 to 20 % faster than one part; above that the two are equal at
  // 128, and at 64 a two-part workgroup fills a unit's registers alone where four one-part ones fit: 2.3 x slower at
  // 8 per unit).  Else one part.  Chains too short to matter stay in one part: more parts want about 64 steps in
  // the longest chain, estimated from the mean sequence length.
  const int64_t blocks64 = (p.k_tokens + 63) / 64 * p.kv_heads, pairs32 = ((p.k_tokens + 31) / 32 + 1) / 2 * p.kv_heads;
  const int64_t longest_chain = p.q_tokens / (p.num_seqs > 0 ? p.num_seqs : 1) / kBmTile * (p.q_heads / p.kv_heads);
  int dkv_parts = 1;
  if (longest_chain >= 64) {
    if (pairs32 <= kBmComputeUnits * 5 / 4) {
      dkv_parts = 4;
    } else if (blocks64 <= (p.head_dim == 128 ? 4 : 2) * kBmComputeUnits) {
      dkv_parts = 2;
    }
  }
  // ARENO_BACKWARD_PARTS=1|2|4 (read at every launch) fixes the choice: the same dK and dV up to the order of the
  // last sums, so this is for tests of the kernels a launch of the test's size would not take, and for timing
  if (const char* e = getenv("ARENO_BACKWARD_PARTS")) {
    if (strcmp(e, "1") == 0) dkv_parts = 1;
    if (strcmp(e, "2") == 0) dkv_parts = 2;
    if (strcmp(e, "4") == 0) dkv_parts = 4;
  }
  // The dq kernel with 32 rows per wave at head dim 128 once the launch has 8 workgroups of 64 rows per compute unit:
  // half the LDS reads per product (4 x 4 096 tokens, 32 / 8 heads: both launches 2 970 -> 2 760 us; 4 x 2 048
  // tokens, 28 / 4 heads: 834 -> 807 us), but half the workgroups and two waves per SIMD instead of three, which
  // costs small launches (8 x 512 tokens: +4 %) and head dim 64 (four waves per SIMD down to two: +5 %).
  // ARENO_BACKWARD_DQ_ROWS=16|32 (read at every launch) fixes the choice, for tests and timing.
  int dq_cb = p.head_dim == 128 && q_blocks * p.q_heads >= 8 * kBmComputeUnits ? 2 : 1;
  if (const char* e = getenv("ARENO_BACKWARD_DQ_ROWS")) {
    if (strcmp(e, "32") == 0) dq_cb = 2;
    if (strcmp(e, "16") == 0) dq_cb = 1;
  }
  const int64_t dq_blocks = (p.q_tokens + kBmRows * dq_cb - 1) / (kBmRows * dq_cb);
  bm_fn dq;
  DkvLaunch dkv;
  if (p.head_dim == 64) {
    dq = dq_cb == 2 ? (bf16 ? bwd_mfma_dq_kernel<KV_BF16, 64, 2> : bwd_mfma_dq_kernel<KV_F16, 64, 2>)
                    : (bf16 ? bwd_mfma_dq_kernel<KV_BF16, 64, 1> : bwd_mfma_dq_kernel<KV_F16, 64, 1>);
    dkv = bf16 ? dkv_launch<KV_BF16, 64>(dkv_parts) : dkv_launch<KV_F16, 64>(dkv_parts);
  } else {
    dq = dq_cb == 2 ? (bf16 ? bwd_mfma_dq_kernel<KV_BF16, 128, 2> : bwd_mfma_dq_kernel<KV_F16, 128, 2>)
                    : (bf16 ? bwd_mfma_dq_kernel<KV_BF16, 128, 1> : bwd_mfma_dq_kernel<KV_F16, 128, 1>);
    dkv = bf16 ? dkv_launch<KV_BF16, 128>(dkv_parts) : dkv_launch<KV_F16, 128>(dkv_parts);
  }
  const char* op = "areno_hip_attention_backward";
  if (dkv.fn == nullptr) return fail(ARENO_ERR_LAUNCH, "%s: the dkv kernel's LDS size was refused", op);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (q_blocks > 0) {
    hipLaunchKernelGGL(dq, dim3(static_cast<unsigned>(dq_blocks * p.q_heads)), dim3(kBmThreads), 0, s, p);
    if (int rc = check_launch(op)) return rc;
  }
  if (k_blocks > 0) {
    const int64_t blocks = (p.k_tokens + dkv.key_rows - 1) / dkv.key_rows;
    const int64_t groups = dkv_parts == 4 ? (blocks + 1) / 2 : blocks;  // (pairs with four parts, see above)
    hipLaunchKernelGGL(dkv.fn, dim3(static_cast<unsigned>(groups * p.kv_heads)), dim3(dkv.threads), dkv.lds_bytes, s, p);
    if (int rc = check_launch(op)) return rc;
  }
  return ARENO_OK;
}

}  // namespace areno
