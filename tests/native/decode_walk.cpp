// CPU walk over the work list of the matrix-core decode kernel: every unit of a launch is taken through the same
// item / cursor functions the kernels use (areno_amd/csrc/decode_items.hpp: the split kernel, the plan kernel and the
// merge kernel), with accessors that check every index before it is used, and every block-table column, cache
// position and partial slot the kernel would touch is checked against the workload; every cached token must be read
// exactly once.  Built by tests/test_decode_walk_cpu.py with g++; no GPU code.
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

// The item table as the kernels hold it: (lo, end, row, nseq) per item and the exclusive prefix sums of the quanta,
// every index checked.
struct CheckedTable {
  const std::vector<ItemInfo>* items;
  const std::vector<int>* cums;
  mutable Fail* fail;
  ItemInfo info(int b) const {
    if (b < 0 || b >= static_cast<int>(items->size())) {
      if (!fail->msg[0]) snprintf(fail->msg, sizeof(fail->msg), "item index %d outside [0, %zu)", b, items->size());
      return ItemInfo{0, 0, 0, 1};
    }
    return (*items)[b];
  }
  int cum(int i) const {
    if (i < 0 || i >= static_cast<int>(cums->size())) {
      if (!fail->msg[0]) snprintf(fail->msg, sizeof(fail->msg), "cum index %d outside [0, %zu)", i, cums->size());
      return 0x3fffffff;
    }
    return (*cums)[i];
  }
};

template <bool GROUPED>
int walk(const ItemShape& shape, const CheckedLens& lens, int units, int tile_tokens, int block_size, int max_blocks,
         long long* quanta_seen, long long* partials, long long* steps, Fail* fail) {
  const int num_items = shape.num_items();
  std::vector<ItemInfo> items(num_items);
  std::vector<int> cum(num_items + 1, 0);
  for (int v = 0; v < num_items; ++v) {
    items[v] = item_info<GROUPED>(shape, lens, v);
    const ItemInfo& it = items[v];
    if (it.quanta() < 0 || (it.end > it.lo && it.lo < 0)) {
      snprintf(fail->msg, sizeof(fail->msg), "item %d has a bad extent [%d, %d)", v, it.lo, it.end);
      return 1;
    }
    cum[v + 1] = cum[v] + it.extent(shape.switch_quanta);
  }
  const CheckedTable table = {&items, &cum, fail};
  const int total = cum[num_items];
  const UnitGeometry geo = make_unit_geometry(total, units);
  // every token of every item must be read exactly once
  std::vector<std::vector<char>> seen(num_items);
  for (int v = 0; v < num_items; ++v) seen[v].assign(items[v].end > items[v].lo ? items[v].end - items[v].lo : 0, 0);
  *partials = 0;
  *steps = 0;
  std::vector<int> written(num_items, 0);  // partials every item got
  for (int unit = 0; unit < units; ++unit) {
    const int q0 = geo.unit_start(unit), q1 = geo.unit_start(unit + 1);
    if (q0 < 0 || q1 > total || q0 > q1) {
      snprintf(fail->msg, sizeof(fail->msg), "unit %d owns [%d, %d) of %d quanta", unit, q0, q1, total);
      return 1;
    }
    if (q0 == q1) continue;
    if (geo.unit_of(q0) != unit || geo.unit_of(q1 - 1) != unit) {
      snprintf(fail->msg, sizeof(fail->msg), "unit_of disagrees with unit_start for unit %d", unit);
      return 1;
    }
    TileCursor c;
    if (!cursor_seek(c, table, shape.switch_quanta, num_items, q0, q1)) continue;  // only switch positions in the unit
    int guard = 0;
    for (;;) {
      if (fail->msg[0]) return 1;
      if (++guard > (1 << 24)) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d: the cursor does not terminate", unit);
        return 1;
      }
      // the cursor is on a tile of item c.b: [c.tok, min(c.tok + tile, c.seg_end))
      if (c.b < 0 || c.b >= num_items) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d: cursor on item %d of %d", unit, c.b, num_items);
        return 1;
      }
      const ItemInfo& it = items[c.b];
      if (c.it.lo != it.lo || c.it.end != it.end || c.it.row != it.row || c.it.nseq != it.nseq) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d: the cursor's copy of item %d differs from the table", unit, c.b);
        return 1;
      }
      if (c.tok < it.lo || c.tok >= c.seg_end || c.seg_end > it.end || c.q_end > q1 || c.q_end > cum[c.b + 1] ||
          c.q_end <= cum[c.b] + shape.switch_quanta || (c.tok - it.lo) % kQuantumTokens != 0) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d item %d: tile at %d, segment end %d (item [%d, %d), q_end %d)",
                 unit, c.b, c.tok, c.seg_end, it.lo, it.end, c.q_end);
        return 1;
      }
      ++*steps;
      const bool shared = GROUPED && c.b < shape.num_shared;
      // rows the tile's pages are read for (a shared item is read through its first row's table for all members)
      const int first_row = it.row, members = it.nseq;
      if (first_row < 0 || first_row + members > shape.batch || members < 1 || members > 16) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d: rows [%d, %d) outside the batch", unit, first_row, first_row + members);
        return 1;
      }
      for (int i = 0; i < tile_tokens; ++i) {
        int t = c.tok + i;
        const bool live = t < c.seg_end;
        if (!live) t = c.seg_end - 1;  // the kernel clamps the lanes behind the segment's end
        const int col = t / block_size;
        for (int m = 0; m < members; ++m) {
          // every member must hold the token (written before this step) and a column for it
          if (t < 0 || t >= lens.row_len(first_row + m) + (shape.append_in_merge ? 0 : 1) || col >= max_blocks) {
            snprintf(fail->msg, sizeof(fail->msg), "unit %d: token %d of row %d (length %d, %d columns)", unit, t,
                     first_row + m, lens.row_len(first_row + m), max_blocks);
            return 1;
          }
        }
        if (live) {
          if (seen[c.b][t - it.lo]) {
            snprintf(fail->msg, sizeof(fail->msg), "token %d of item %d read twice", t, c.b);
            return 1;
          }
          seen[c.b][t - it.lo] = 1;
        }
      }
      const int b_before = c.b;
      const CursorMove mv = cursor_advance(c, table, shape.switch_quanta, q1, tile_tokens);
      if (mv != kCursorSameSegment) {
        // the segment is done: one partial, into slot unit + row (or unit + item)
        const long long slot = static_cast<long long>(unit) + (shared ? b_before : first_row);
        const long long slots = static_cast<long long>(units) + (shared ? shape.num_shared : shape.batch);
        if (slot < 0 || slot >= slots) {
          snprintf(fail->msg, sizeof(fail->msg), "unit %d: partial slot %lld outside [0, %lld)", unit, slot, slots);
          return 1;
        }
        ++*partials;
        ++written[b_before];
        // the merge kernel finds the partial through unit_of over the item's quanta
        int u_lo, u_hi;
        item_units(geo, shape.switch_quanta, cum[b_before], cum[b_before + 1], u_lo, u_hi);
        if (unit < u_lo || unit > u_hi) {
          snprintf(fail->msg, sizeof(fail->msg), "unit %d wrote a partial of item %d, whose units are [%d, %d]", unit,
                   b_before, u_lo, u_hi);
          return 1;
        }
      }
      if (mv == kCursorUnitDone) break;
      if (mv == kCursorOpensItem && c.b <= b_before) {
        snprintf(fail->msg, sizeof(fail->msg), "unit %d: the cursor went from item %d to item %d", unit, b_before, c.b);
        return 1;
      }
    }
  }
  for (int v = 0; v < num_items; ++v) {
    for (size_t i = 0; i < seen[v].size(); ++i) {
      if (!seen[v][i]) {
        snprintf(fail->msg, sizeof(fail->msg), "token %zu of item %d was never read", items[v].lo + i, v);
        return 1;
      }
    }
  }
  // the merge kernel reads one partial from every unit of an item's range: each of them must have written one
  for (int v = 0; v < num_items; ++v) {
    int expected = 0;
    if (items[v].quanta() > 0) {
      int u_lo, u_hi;
      item_units(geo, shape.switch_quanta, cum[v], cum[v + 1], u_lo, u_hi);
      expected = u_hi - u_lo + 1;
    }
    if (written[v] != expected) {
      snprintf(fail->msg, sizeof(fail->msg), "item %d got %d partials, the merge reads %d", v, written[v], expected);
      return 1;
    }
  }
  *quanta_seen = 0;
  for (int v = 0; v < num_items; ++v) *quanta_seen += items[v].quanta();
  return fail->msg[0] ? 1 : 0;
}

}  // namespace

extern "C" int decode_walk(const int32_t* cache_seqlens, int batch, const int32_t* shared_lens, int group_rows,
                           int q_per_kv, int window_left, int append_in_merge, int switch_quanta, int units,
                           int tile_tokens,
                           int block_size, int max_blocks, long long* quanta_seen, long long* partials,
                           long long* steps, char* message, int message_bytes) {
  Fail fail;
  fail.msg[0] = 0;
  ItemShape shape = {batch, window_left, append_in_merge, switch_quanta, 0, 1, 1, 1};
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
  const int rc = num_shared > 0 ? walk<true>(shape, lens, units, tile_tokens, block_size, max_blocks, quanta_seen,
                                             partials, steps, &fail)
                                : walk<false>(shape, lens, units, tile_tokens, block_size, max_blocks, quanta_seen,
                                              partials, steps, &fail);
  if (message != nullptr && message_bytes > 0) {
    strncpy(message, fail.msg, message_bytes - 1);
    message[message_bytes - 1] = 0;
  }
  return rc;
}
