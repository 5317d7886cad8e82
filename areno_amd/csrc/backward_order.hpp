// The order in which the workgroups of the matrix-core backward kernels (attention_backward_mfma.hip) take the blocks
// of packed rows; host and device code, so that a CPU test can walk it (tests/native/backward_order.cpp).
#pragma once

#include <stdint.h>

#include "decode_items.hpp"  // ARENO_HD

namespace areno {

// The block of packed rows the i-th workgroup (of a head) takes.  Blocks differ in cost by their place in their
// sequence (a query block late in a long sequence sees the most keys, a key block early in it is seen by the most
// queries), and a launch ends soonest when the expensive blocks start first.  The lengths are not known on the host,
// so the order assumes sequences of about equal length: the packed blocks are cut into num_seqs runs and taken run by
// run in turn, the expensive end of every run first (`from_end`: the last block of a run).  Any order is correct.
ARENO_HD int64_t block_in_cost_order(int64_t i, int64_t blocks, int num_seqs, bool from_end) {
  const int64_t runs = num_seqs > 0 ? num_seqs : 1, per = blocks / runs, rest = blocks - per * runs;
  if (per == 0) return from_end ? blocks - 1 - i : i;
  if (from_end) {  // the blocks behind the last whole run belong to the end of the last sequence: first
    if (i < rest) return blocks - 1 - i;
    const int64_t j = i - rest;
    return (j % runs) * per + (per - 1 - j / runs);
  }
  if (i >= per * runs) return i;
  return (i % runs) * per + i / runs;
}

}  // namespace areno
