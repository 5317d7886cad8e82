// Work list of the matrix-core decode kernel: how a batch becomes items, items become quanta of 16 tokens, and the
// quantum range is cut into units of equal cost, one per wave.  Plain C++ shared by the split kernel, the merge
// kernel, the plan kernel and the host (the launcher sizes the workspace with it, and a CPU test walks every unit of
// a workload through the same functions and checks each index they produce before anything is loaded through it).
//
// Items.  Without prefix groups item v is row v: the cached keys the row's query may see, [first_allowed, end), the
// reference's range (areno/accel/csrc/attention.cu:588-604) with end = L_v + 1 when the token being appended is in
// its page already and end = L_v when the merge launch folds that token in (it is not in the page yet).  With
// prefix groups the list is
//   [shared prefix of every sub-group of rows that sit side by side in the 16 matrix-core columns]
//   + [the rest of every row],
// a shared item being read once for all rows of its sub-group.  An item may be empty (a row without cached keys).
// Quanta.  An item is ceil((end - lo) / 16) quanta of 16 tokens, the last one possibly short.
// Cost line.  The items lie one behind the other on a line of cost positions: a non-empty item takes
// switch_quanta positions that carry no tokens (what it costs a wave to change items: a partial, the next Q, the
// softmax state) and then one position per quantum.  Unit u owns positions [u * total / units, (u + 1) * total /
// units): every unit has the same cost to within one position.  The part of an item inside a unit is a segment; a
// wave goes through a segment in tile steps of 32 or 64 tokens counted from the segment's first token, the last step
// masked at the segment's end.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define ARENO_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define ARENO_HD inline
#endif

namespace areno {

constexpr int kTileTokens = 32;      // key tile of the prefill kernel; shared prefix lengths are cut to multiples of it
constexpr int kQuantumTokens = 16;   // granularity of the decode kernel's unit borders
constexpr int kMfmaMaxBatch = 1024;  // rows one launch indexes: the prefix sum over the items lives in LDS

// first key a query at position length - 1 may see (window_left < 0: no window)
ARENO_HD int first_visible_key(int length, int window_left) {
  if (window_left < 0) return 0;
  const int lo = length - 1 - window_left;
  return lo > 0 ? lo : 0;
}

struct UnitGeometry {
  int total;  // cost positions of the launch
  int units;  // units that own positions: the launch's units, or only as many as there are positions (see below)
  bool narrow;  // the products below fit 32 bits: 32-bit divisions are a fifth of the instructions of 64-bit ones

  ARENO_HD int unit_start(int u) const {
    if (u >= units) return total;  // a unit behind the last one that owns positions
    if (narrow)
      return static_cast<int>(static_cast<uint32_t>(u) * static_cast<uint32_t>(total) / static_cast<uint32_t>(units));
    return static_cast<int>(static_cast<long long>(u) * total / units);
  }
  // unit that owns position x, 0 <= x < total: the largest u with unit_start(u) <= x
  ARENO_HD int unit_of(int x) const {
    if (narrow)
      return static_cast<int>((static_cast<uint32_t>(x + 1) * static_cast<uint32_t>(units) +
                               static_cast<uint32_t>(total) - 1u) /
                              static_cast<uint32_t>(total)) -
             1;
    return static_cast<int>((static_cast<long long>(x + 1) * units + total - 1) / total - 1);
  }
};

// A launch with fewer than two cost positions per unit (a tiny batch) uses only its first total / 2 units, two
// positions each (a tile step reads two quanta of tokens anyway), and leaves the others without work: spread over
// all units, a row's positions would lie in units far apart with empty ones in between, and the merge would go
// through the whole range (256 candidates for a single row of any length).
ARENO_HD UnitGeometry make_unit_geometry(int total, int units) {
  UnitGeometry g;
  g.total = total;
  g.units = total < 2 * units ? (total > 1 ? total / 2 : 1) : units;
  // largest product in unit_start / unit_of: (total + 1) * units + total
  g.narrow = (static_cast<long long>(total) + 2) * (static_cast<long long>(units) + 1) < (1LL << 31);
  return g;
}

// How the rows of a launch become items.
struct ItemShape {
  int batch;
  int window_left;
  int append_in_merge;  // 1: the token being appended is not in its page; items end in front of it (the merge adds it)
  int switch_quanta;    // cost positions in front of a non-empty item's quanta
  // prefix groups; num_shared = 0 and the other three = 1 without them
  int num_shared;      // shared items, listed in front of the per-row items
  int group_rows;      // rows per prefix group
  int cols_seqs;       // rows that fit side by side: 16 / (q heads per kv head)
  int subs_per_group;  // ceil(group_rows / cols_seqs)

  ARENO_HD int num_items() const { return num_shared + batch; }
  ARENO_HD int num_groups() const { return group_rows > 0 ? batch / group_rows : 0; }
};

struct ItemInfo {
  int lo;    // first token
  int end;   // end of the cached tokens the item reads through the block table of `row`
  int row;   // block-table / query row (first row of the sub-group for a shared item)
  int nseq;  // rows served side by side (1 for a per-row item)
  ARENO_HD int quanta() const { return end > lo ? (end - lo + kQuantumTokens - 1) / kQuantumTokens : 0; }
  // positions on the cost line
  ARENO_HD int extent(int switch_quanta) const { return end > lo ? quanta() + switch_quanta : 0; }
};

// Lens supplies  int row_len(int row)  (cache_seqlens)  and  int group_len(int group)  (shared_prefix_lens).
// Tokens of a sub-group's shared prefix: the caller's figure, clipped to what every member has cached and cut to a
// whole number of 32-token tiles.
template <class Lens>
ARENO_HD int shared_prefix_tokens(const ItemShape& s, const Lens& lens, int sub, int& row0, int& count) {
  const int gi = sub / s.subs_per_group;
  const int j = sub - gi * s.subs_per_group;
  row0 = gi * s.group_rows + j * s.cols_seqs;
  const int left = s.group_rows - j * s.cols_seqs;
  count = s.cols_seqs < left ? s.cols_seqs : left;
  int len = lens.group_len(gi);
  for (int m = 0; m < count; ++m) {
    const int l = lens.row_len(row0 + m);
    len = l < len ? l : len;
  }
  return (len > 0 ? len : 0) & ~(kTileTokens - 1);
}

template <bool GROUPED, class Lens>
ARENO_HD ItemInfo item_info(const ItemShape& s, const Lens& lens, int v) {
  ItemInfo it = {0, 0, 0, 1};
  if constexpr (GROUPED) {
    if (v < s.num_shared) {
      it.end = shared_prefix_tokens(s, lens, v, it.row, it.nseq);
      return it;
    }
    const int b = v - s.num_shared;
    const int gi = b / s.group_rows;
    int row0, count;
    it.lo = shared_prefix_tokens(s, lens, gi * s.subs_per_group + (b - gi * s.group_rows) / s.cols_seqs, row0, count);
    it.end = lens.row_len(b) + 1 - s.append_in_merge;
    it.row = b;
    return it;
  } else {
    const int len = lens.row_len(v);
    it.lo = first_visible_key(len + 1, s.window_left);
    it.end = len + 1 - s.append_in_merge;
    it.row = v;
    return it;
  }
}

// Position of a wave's tile stream: the item, the first token of the tile, and where the segment (the part of the
// item that belongs to the wave's unit) ends.
struct TileCursor {
  int b;
  int tok;
  int seg_end;  // end of the segment in tokens (<= it.end)
  int q_end;    // end of the segment on the cost line: min(cum(b + 1), end of the unit)
  ItemInfo it;
};

enum CursorMove { kCursorSameSegment = 0, kCursorOpensItem = 1, kCursorUnitDone = 2 };

// Table supplies  ItemInfo info(int b)  and  int cum(int i)  = cost positions of items [0, i), 0 <= i <= num_items.
// Put the cursor on the part of item b (non-empty, cum(b) <= from < cum(b + 1)) that lies in [from, c1); false when
// that part holds no quantum (c1 does not reach past the item's switch positions).
template <class Table>
ARENO_HD bool cursor_open(TileCursor& c, const Table& t, int switch_quanta, int b, int from, int c1) {
  const int first = t.cum(b) + switch_quanta;  // position of the item's first quantum
  if (c1 <= first) return false;
  c.b = b;
  c.it = t.info(b);
  const int ce = t.cum(b + 1);
  c.q_end = ce < c1 ? ce : c1;
  const int start = from > first ? from : first;
  c.tok = c.it.lo + (start - first) * kQuantumTokens;
  const int e = c.it.lo + (c.q_end - first) * kQuantumTokens;
  c.seg_end = e < c.it.end ? e : c.it.end;
  return true;
}

// Put the cursor on the first tile of the unit [c0, c1), 0 <= c0 < c1 <= cum(num_items); false when the unit holds
// no quantum.
template <class Table>
ARENO_HD bool cursor_seek(TileCursor& c, const Table& t, int switch_quanta, int num_items, int c0, int c1) {
  int lo = 0, hi = num_items;
  while (lo + 1 < hi) {  // the largest item index with cum <= c0; empty items in front of it are skipped
    const int mid = (lo + hi) >> 1;
    if (t.cum(mid) <= c0) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return cursor_open(c, t, switch_quanta, lo, c0, c1);
}

// The next non-empty item behind position q = cum(b + 1) of item b, when the unit [.., c1) reaches its quanta;
// -1 otherwise.  (q < c1 <= cum(num_items), so a non-empty item follows.)
template <class Table>
ARENO_HD int next_item_in_unit(const Table& t, int switch_quanta, int b, int q, int c1) {
  if (q >= c1) return -1;
  int n = b + 1;
  while (t.cum(n + 1) == q) ++n;  // empty items
  return c1 > q + switch_quanta ? n : -1;
}

// Move the cursor one tile step of `tile_tokens` tokens on inside the unit that ends at position c1.
template <class Table>
ARENO_HD CursorMove cursor_advance(TileCursor& c, const Table& t, int switch_quanta, int c1, int tile_tokens) {
  c.tok += tile_tokens;
  if (c.tok < c.seg_end) return kCursorSameSegment;
  const int q = c.q_end;
  const int n = next_item_in_unit(t, switch_quanta, c.b, q, c1);
  if (n < 0) return kCursorUnitDone;
  cursor_open(c, t, switch_quanta, n, q, c1);
  return kCursorOpensItem;
}

// Units that hold quanta of an item with cost positions [cb, ce) (ce > cb): the first and the last.
ARENO_HD void item_units(const UnitGeometry& geo, int switch_quanta, int cb, int ce, int& first, int& last) {
  first = geo.unit_of(cb + switch_quanta);
  last = geo.unit_of(ce - 1);
}

// Sub-groups of a prefix group that sit side by side in the 16 matrix-core columns, or 0 when grouping does not apply.
inline int shared_items_for(int batch, int group, int group_rows, int* cols_seqs, int* subs_per_group) {
  const int cs = group > 0 ? 16 / group : 0;
  if (group_rows < 2 || cs < 2 || batch % group_rows != 0) return 0;
  *cols_seqs = cs;
  *subs_per_group = (group_rows + cs - 1) / cs;
  return batch / group_rows * *subs_per_group;
}

}  // namespace areno
