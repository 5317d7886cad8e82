// CPU walk of the block order of the matrix-core backward kernels (areno_amd/csrc/backward_order.hpp): every order is
// a permutation of the blocks, and for sequences of equal length the blocks come by cost (all sequences' most
// expensive block first, then the next, ...).  Built by tests/test_backward_order_cpu.py with g++.
#include <stdio.h>

#include <vector>

#include "../../areno_amd/csrc/backward_order.hpp"

extern "C" int backward_order_check(int max_blocks, int max_seqs, long long* cases, char* msg, int msg_len) {
  *cases = 0;
  for (int blocks = 1; blocks <= max_blocks; ++blocks) {
    for (int seqs = 0; seqs <= max_seqs; ++seqs) {
      for (int from_end = 0; from_end < 2; ++from_end) {
        ++*cases;
        std::vector<int> seen(blocks, 0);
        long long last_place = -1;
        for (int i = 0; i < blocks; ++i) {
          const long long b = areno::block_in_cost_order(i, blocks, seqs, from_end != 0);
          if (b < 0 || b >= blocks || seen[b]++) {
            snprintf(msg, msg_len, "blocks %d seqs %d from_end %d: workgroup %d takes block %lld (outside or twice)",
                     blocks, seqs, from_end, i, b);
            return 1;
          }
          if (seqs > 0 && blocks % seqs == 0) {
            // equal sequences of blocks / seqs blocks each: the place inside the sequence, counted from the expensive
            // end, never goes down
            const long long per = blocks / seqs, in_run = b % per, place = from_end ? per - 1 - in_run : in_run;
            if (place < last_place) {
              snprintf(msg, msg_len, "blocks %d seqs %d from_end %d: workgroup %d takes place %lld after %lld", blocks,
                       seqs, from_end, i, place, last_place);
              return 1;
            }
            last_place = place;
          }
        }
      }
    }
  }
  return 0;
}
