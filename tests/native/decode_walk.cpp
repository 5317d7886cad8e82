// CPU walk over the work list of the matrix-core decode kernel: every unit of a launch is taken through the same
// item / cursor functions the kernel uses (areno_amd/csrc/decode_items.hpp), with accessors that check every index
// before it is used, and every block-table column, cache position and partial slot the kernel would touch is checked
// against the workload.  Built by tests/test_decode_walk_cpu.py with g++; no GPU code.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "../../areno_amd/csrc/decode_items.hpp"

using namespace areno;

namespace {

struct Fail {
  char msg[256];
};

struct CheckedLens {
  const int32_t* len;
  int batch;
  const int32_t* glen;
  int groups;
  mutable Fail* fail;
  int row_len(int b) const {
    if (b < 0 || b >= batch) {
      if (!fail->msg[0]) snprintf(fail->msg, sizeof(fail->msg), "row_len index %d outside [0, %d)", b, batch);
      return 0;
    }
    return len[b];
  }
  int group_len(int g) const {
    if (g < 0 || g >= groups) {
      if (!fail->msg[0]) snprintf(fail->msg, sizeof(fail->msg), "group_len index %d outside [0, %d)", g, groups);
      return 0;
    }
    return glen[g];
  }
};

struct CheckedCum {
  const std::vector<int>* cum;
  mutable Fail* fail;
  int at(int i) const {
    if (i < 0 || i >= static_cast<int>(cum->size())) {
      if (!fail->msg[0]) snprintf(fail->msg, sizeof(fail->msg), "cum index %d outside [0, %zu)", i, cum->size());
      return 0x3fffffff;
    }
    return (*cum)[i];
  }
};

template <bool GROUPED>
int walk(const ItemShape& shape, const CheckedLens& lens, int units, int block_size, int max_blocks, long long* tiles_seen,
         long long* partials, Fail* fail) {
  const int num_items = shape.num_items();
  std::vector<int> cum(num_items + 1, 0);
  for (int v = 0; v < num_items; ++v) {
    const ItemInfo it = item_info<GROUPED>(shape, lens, v);
    if (it.end < it.lo || it.tiles() < 0) {
      snprintf(fail->msg, sizeof(fail->msg), "item %d has a negative extent [%d, %d)", v, it.lo, it.end);
      return 1;
    }
    cum[v + 1] = cum[v] + it.tiles();
  }
  const CheckedCum ccum = {&cum, fail};
  const int total = cum[num_items];
  const UnitGeometry geo = make_unit_geometry(total, units);
  std::vector<int> visits(total, 0);
  *partials = 0;
  for (int unit = 0; unit < units; ++unit) {
    const int x0 = geo.unit_start(unit), x1 = geo.unit_start(unit + 1);
    if (x0 < 0 || x1 > total || x0 > x1) {
      snprintf(fail->msg, sizeof(fail->msg), "unit %d owns [%d, %d) of %d tiles", unit, x0, x1, total);
      return 1;
    }
    if (x0 == x1) continue;
    if (geo.unit_of(x0) != unit || geo.unit_of(x1 - 1) != unit) {
      snprintf(fail->msg, sizeof(fail->msg), "unit_of disagrees with unit_start for unit %d", unit);
      return 1;
    }
    TileCursor c;
    cursor_seek<GROUPED>(c, shape, lens, ccum, x0);
    for (int x = x0; x < x1; ++x) {
      bool opens = x == x0;
      if (x > x0) opens = cursor_advance<GROUPED>(c, shape, lens, ccum, x);
      if (fail->msg[0]) return 1;
      if (c.b < 0 || c.b >= num_items || x < cum[c.b] || x >= cum[c.b + 1]) {
        snprintf(fail->msg, sizeof(fail->msg), "tile %d: cursor on item %d, which owns [%d, %d)", x, c.b,
                 c.b >= 0 && c.b < num_items ? cum[c.b] : -1, c.b >= 0 && c.b < num_items ? cum[c.b + 1] : -1);
        return 1;
      }
      if (c.tok != c.it.lo + (x - cum[c.b]) * kTileTokens) {
        snprintf(fail->msg, sizeof(fail->msg), "tile %d: cursor token %d, expected %d", x, c.tok,
                 c.it.lo + (x - cum[c.b]) * kTileTokens);
        return 1;
      }
      ++visits[x];
      const bool shared = GROUPED && c.b < shape.num_shared;
      // rows the tile's pages are read for (a shared item is read through its first row's table for all members)
      const int first_row = c.it.row, members = c.it.nseq;
      if (first_row < 0 || first_row + members > shape.batch || members < 1 || members > 16) {
        snprintf(fail->msg, sizeof(fail->msg), "tile %d: rows [%d, %d) outside the batch", x, first_row, first_row + members);
        return 1;
      }
      if (c.on_new_token()) {
        if (shared || !c.it.has_new || c.tok - c.it.end >= kTileTokens || x != cum[c.b + 1] - 1) {
          snprintf(fail->msg, sizeof(fail->msg), "tile %d: unexpected new-token tile (item %d tok %d end %d)", x, c.b, c.tok, c.it.end);
          return 1;
        }
        // the token goes to position L of the row: its column must exist
        const int pos = c.it.end;
        if (pos != lens.row_len(first_row) || pos / block_size >= max_blocks) {
          snprintf(fail->msg, sizeof(fail->msg), "tile %d: append position %d of row %d (length %d, %d columns)", x, pos,
                   first_row, lens.row_len(first_row), max_blocks);
          return 1;
        }
      } else {
        for (int i = 0; i < kTileTokens; ++i) {
          int t = c.tok + i;
          if (t > c.it.end - 1) t = c.it.end - 1;  // the kernel clamps the lanes behind the item's end
          const int col = t / block_size;
          for (int m = 0; m < members; ++m) {
            // every member must hold the token (written before this step) and a column for it
            if (t < 0 || t >= lens.row_len(first_row + m) + (shape.new_token_tile ? 0 : 1) || col >= max_blocks) {
              snprintf(fail->msg, sizeof(fail->msg), "tile %d: token %d of row %d (length %d, %d columns)", x, t,
                       first_row + m, lens.row_len(first_row + m), max_blocks);
              return 1;
            }
          }
        }
      }
      // a partial is written when the unit ends or the next tile opens an item: slot unit + row (or unit + item)
      const bool last = x + 1 == x1;
      bool next_opens = false;
      if (!last) next_opens = x + 1 == c.x_end;
      if (last || next_opens) {
        const long long slot = static_cast<long long>(unit) + (shared ? c.b : first_row);
        const long long slots = static_cast<long long>(units) + (shared ? shape.num_shared : shape.batch);
        if (slot < 0 || slot >= slots) {
          snprintf(fail->msg, sizeof(fail->msg), "tile %d: partial slot %lld outside [0, %lld)", x, slot, slots);
          return 1;
        }
        ++*partials;
      }
      (void)opens;
    }
  }
  for (int x = 0; x < total; ++x) {
    if (visits[x] != 1) {
      snprintf(fail->msg, sizeof(fail->msg), "tile %d visited %d times", x, visits[x]);
      return 1;
    }
  }
  *tiles_seen = total;
  return fail->msg[0] ? 1 : 0;
}

}  // namespace

extern "C" int decode_walk(const int32_t* cache_seqlens, int batch, const int32_t* shared_lens, int group_rows,
                           int q_per_kv, int window_left, int new_token_tile, int units, int block_size, int max_blocks,
                           long long* tiles_seen, long long* partials, char* message, int message_bytes) {
  Fail fail;
  fail.msg[0] = 0;
  ItemShape shape = {batch, window_left, new_token_tile, 0, 1, 1, 1};
  int cols = 0, subs = 0;
  int num_shared = 0;
  if (shared_lens != nullptr && window_left < 0) num_shared = shared_items_for(batch, q_per_kv, group_rows, &cols, &subs);
  if (num_shared > 0) {
    shape.num_shared = num_shared;
    shape.group_rows = group_rows;
    shape.cols_seqs = cols;
    shape.subs_per_group = subs;
  }
  const CheckedLens lens = {cache_seqlens, batch, shared_lens, num_shared > 0 ? batch / group_rows : 0, &fail};
  const int rc = num_shared > 0 ? walk<true>(shape, lens, units, block_size, max_blocks, tiles_seen, partials, &fail)
                                : walk<false>(shape, lens, units, block_size, max_blocks, tiles_seen, partials, &fail);
  if (message != nullptr && message_bytes > 0) {
    strncpy(message, fail.msg, message_bytes - 1);
    message[message_bytes - 1] = 0;
  }
  return rc;
}
