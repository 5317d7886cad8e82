// CPU check of the prefill kernel's step geometry (areno_amd/csrc/prefill_steps.hpp): the closed forms for the tile
// steps in front of a query block and the bisection that finds the block of a step, held against a walk over the
// blocks with block_tiles(), the one definition of which key tiles a block sees.  Built by
// tests/test_prefill_steps_cpu.py with g++; no GPU code.
#include <stdint.h>
#include <stdio.h>

#include "../../areno_amd/csrc/prefill_steps.hpp"

using namespace areno;

// Checks one sequence shape; returns 0 or writes what differs.  `every_step` also places every step of the sequence
// (quadratic in the sequence's size: for small shapes).
extern "C" int prefill_steps_check(int n_new, int ctx, int tq, int window_left, int every_step, long long* steps_out,
                                   char* msg, int msg_len) {
  const int blocks = query_blocks(n_new, tq);
  long long walked = 0;
  for (int j = 0; j <= blocks; ++j) {
    const int closed = steps_before_block(n_new, ctx, j, tq, window_left);
    if (closed != walked) {
      snprintf(msg, msg_len, "steps_before_block(n_new=%d, ctx=%d, j=%d, tq=%d, window=%d) = %d, the walk gives %lld",
               n_new, ctx, j, tq, window_left, closed, walked);
      return 1;
    }
    if (j == blocks) break;
    const BlockTiles b = block_tiles(n_new, ctx, j, tq, window_left);
    if (b.count() < 1 || b.cnt < 1 || b.tile_lo < 0) {
      snprintf(msg, msg_len, "block_tiles(n_new=%d, ctx=%d, j=%d, tq=%d, window=%d): count %d, tokens %d, tile_lo %d",
               n_new, ctx, j, tq, window_left, b.count(), b.cnt, b.tile_lo);
      return 1;
    }
    // the block of a step: the block's first and last step always, every step on request
    for (int k = 0; k < b.count(); k = (every_step || k == b.count() - 1) ? k + 1 : b.count() - 1) {
      const int off = static_cast<int>(walked) + k;
      const int found = block_of_step(n_new, ctx, tq, window_left, off);
      if (found != j) {
        snprintf(msg, msg_len, "block_of_step(n_new=%d, ctx=%d, tq=%d, window=%d, off=%d) = %d, the walk gives %d",
                 n_new, ctx, tq, window_left, off, found, j);
        return 1;
      }
    }
    walked += b.count();
  }
  if (sequence_steps(n_new, ctx, tq, window_left) != walked) {
    snprintf(msg, msg_len, "sequence_steps(n_new=%d, ctx=%d, tq=%d, window=%d) differs from the walk", n_new, ctx, tq,
             window_left);
    return 1;
  }
  *steps_out = walked;
  return 0;
}

// The same over a grid: n_new in [0, n_hi], ctx in [0, ctx_hi], every tq and window given.
extern "C" int prefill_steps_check_grid(int n_hi, int ctx_hi, const int* tqs, int num_tq, const int* windows,
                                        int num_windows, long long* shapes_out, char* msg, int msg_len) {
  long long shapes = 0, steps = 0;
  for (int t = 0; t < num_tq; ++t)
    for (int w = 0; w < num_windows; ++w)
      for (int ctx = 0; ctx <= ctx_hi; ++ctx)
        for (int n = 0; n <= n_hi; ++n) {
          if (prefill_steps_check(n, ctx, tqs[t], windows[w], 1, &steps, msg, msg_len)) return 1;
          ++shapes;
        }
  *shapes_out = shapes;
  return 0;
}
