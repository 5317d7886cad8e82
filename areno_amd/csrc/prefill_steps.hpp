// Tile steps of the prefill kernel's work list: a sequence's new tokens are cut into query blocks of tq tokens
// (at least 4; a power of two unless the q heads of a kv head are not), block j may see the key tiles [tile_lo, tile_hi] of kTileTokens keys, and the blocks'
// tile steps lie one behind the other on the line the launch shares out in equal ranges.  Plain C++ shared by the
// prefill kernel, its merge kernel and a CPU test that holds the closed forms below against a walk over the blocks.
//
// The number of steps in front of a block is needed by every workgroup at its start (the prefix sum over the
// sequences and the place of the workgroup's first step), so it is a closed form, not a loop over the blocks: a
// sequence of 4 096 new tokens has 64 to 1 024 blocks, and the thread that walked them alone kept its workgroup --
// every workgroup of the launch -- waiting for 10-25 us.
#pragma once

#include <stdint.h>

#include "decode_items.hpp"

namespace areno {

// Key tiles query block j (tokens [j * tq, ...)) of a sequence may see: [tile_lo, tile_hi].
struct BlockTiles {
  int tok0, cnt, tile_lo, tile_hi;
  ARENO_HD int count() const { return tile_hi - tile_lo + 1; }
};

ARENO_HD BlockTiles block_tiles(int n_new, int ctx, int j, int tq, int window_left) {
  BlockTiles b;
  b.tok0 = j * tq;
  b.cnt = tq < n_new - b.tok0 ? tq : n_new - b.tok0;
  const int key_hi = ctx + b.tok0 + b.cnt - 1;
  const int key_lo_raw = ctx + b.tok0 - window_left;
  const int key_lo = window_left >= 0 ? (key_lo_raw > 0 ? key_lo_raw : 0) : 0;
  b.tile_lo = key_lo / kTileTokens;
  b.tile_hi = key_hi / kTileTokens;
  return b;
}

// Division of a non-negative value by the block size: a shift for the usual power of two.
ARENO_HD bool is_power_of_two(int x) { return (x & (x - 1)) == 0; }
ARENO_HD int div_block(int x, int tq) {
  return is_power_of_two(tq) ? x >> __builtin_ctz(static_cast<unsigned>(tq)) : x / tq;
}
ARENO_HD int query_blocks(int n_new, int tq) { return div_block(n_new + tq - 1, tq); }

constexpr int kTileShift = 5;
static_assert((1 << kTileShift) == kTileTokens, "tile size");

// sum over i in [0, n) of floor(i / r), r = 2^r_shift
ARENO_HD long long floor_ramp(long long n, int r_shift) {
  const long long q = n >> r_shift;
  return ((q * (q - 1) / 2) << r_shift) + q * (n - (q << r_shift));
}

// sum over j in [0, n) of floor((a + j * tq) / kTileTokens) for a >= 0.
// A power of two is either a multiple of the tile (every block adds tq / kTileTokens whole tiles) or divides it
// (r = kTileTokens / tq blocks per tile: floor((a + j * tq) / kTileTokens) = floor((floor(a / tq) + j) / r)).
// Any other block size (a group of q heads that is no power of two folds 256 / group tokens into a block): with
// a = 32 A + a0 and tq = 32 W + r the term is A + j W + floor((a0 + j r) / 32), and the last part repeats, up to a
// constant, with period P = 32 / gcd(r, 32) in j: term(j + P) = term(j) + P r / 32.  One period is summed in a loop of
// at most 32 steps; no division by a run-time value anywhere (a 64-bit one costs a GPU thread some hundred
// instructions, and the bisection below evaluates several sums per step).
ARENO_HD long long tile_index_sum(long long a, int tq, long long n) {
  if (n <= 0) return 0;
  if (is_power_of_two(tq)) {
    const int tq_shift = __builtin_ctz(static_cast<unsigned>(tq));
    if (tq_shift >= kTileShift) return n * (a >> kTileShift) + ((n * (n - 1) / 2) << (tq_shift - kTileShift));
    const int r_shift = kTileShift - tq_shift;
    const long long c = a >> tq_shift;
    return floor_ramp(c + n, r_shift) - floor_ramp(c, r_shift);
  }
  const int r = tq & (kTileTokens - 1), a0 = static_cast<int>(a & (kTileTokens - 1));
  long long sum = n * (a >> kTileShift) + (tq >> kTileShift) * (n * (n - 1) / 2);
  if (r == 0) return sum;
  const int g_shift = __builtin_ctz(static_cast<unsigned>(r));  // gcd(r, 32) = 2^g_shift, the lowest set bit of r
  const int p_shift = kTileShift - g_shift;                     // period P = 2^p_shift
  const int inc = r >> g_shift;                                 // P r / 32
  const long long q = n >> p_shift;
  const int rest = static_cast<int>(n - (q << p_shift));
  int period_sum = 0, rest_sum = 0;
  for (int j = 0; j < (1 << p_shift); ++j) {
    const int term = (a0 + j * r) >> kTileShift;
    period_sum += term;
    if (j < rest) rest_sum += term;
  }
  return sum + q * period_sum + ((inc * (q * (q - 1) / 2)) << p_shift) + rest_sum + rest * q * inc;
}

// Tile steps of blocks [0, j) of a sequence, 0 <= j <= query_blocks(n_new, tq): the sum of block_tiles(...).count().
// tile_hi of a block that is not the sequence's last is floor((ctx + (i + 1) * tq - 1) / kTileTokens), of the last
// floor((ctx + n_new - 1) / kTileTokens); tile_lo is 0 up to the first block whose lowest visible key
// ctx + i * tq - window_left lies beyond key 0.
ARENO_HD int steps_before_block(int n_new, int ctx, int j, int tq, int window_left) {
  if (j <= 0) return 0;
  const int blocks = query_blocks(n_new, tq);
  const int full = j < blocks ? j : blocks - 1;
  long long sum = tile_index_sum(static_cast<long long>(ctx) + tq - 1, tq, full);
  if (j >= blocks) sum += (static_cast<long long>(ctx) + n_new - 1) >> kTileShift;
  if (window_left >= 0) {
    const int j0 = ctx > window_left ? 0 : div_block(window_left - ctx, tq) + 1;
    if (j0 < j) {
      sum -= tile_index_sum(static_cast<long long>(ctx) - window_left + static_cast<long long>(j0) * tq, tq, j - j0);
    }
  }
  return static_cast<int>(sum + j);
}

ARENO_HD int sequence_steps(int n_new, int ctx, int tq, int window_left) {
  return steps_before_block(n_new, ctx, query_blocks(n_new, tq), tq, window_left);
}

// The block that holds step `off` of a sequence, 0 <= off < sequence_steps(...): every block has at least one step
// (a query sees itself), so the steps in front of a block grow strictly with the block and a bisection finds it.
ARENO_HD int block_of_step(int n_new, int ctx, int tq, int window_left, int off) {
  int lo = 0, hi = query_blocks(n_new, tq);
  while (lo + 1 < hi) {
    const int mid = (lo + hi) >> 1;
    if (steps_before_block(n_new, ctx, mid, tq, window_left) <= off) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

}  // namespace areno
