// Work list of the matrix-core decode kernel: how a batch becomes items, items become 32-token tiles, and the
// tile range is cut into equal units, one per wave.  Plain C++ shared by the split kernel, the merge kernel and the
// host (the launcher sizes the workspace with it, and a CPU test walks every unit of a workload through the same
// functions and checks each index they produce before anything is loaded through it).
//
// Items.  Without prefix groups item v is row v: its visible keys [first_allowed, L_v] (the reference's range,
// areno/accel/csrc/attention.cu:588-604).  With prefix groups the list is
//   [shared prefix of every sub-group of rows that sit side by side in the 16 matrix-core columns]
//   + [the rest of every row],
// a shared item being read once for all rows of its sub-group.
// Tiles.  An item is ceil((end - lo) / 32) regular tiles of cached tokens; when the append rides along (the newest
// token's K / V row is not in the page yet) a per-row item ends in one more tile that holds only that token, taken
// from the update row.
// Units.  Unit u owns tiles [u * total / units, (u + 1) * total / units).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define ARENO_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define ARENO_HD inline
#endif

namespace areno {

constexpr int kTileTokens = 32;
constexpr int kMfmaMaxBatch = 1024;  // rows one launch indexes: the prefix sum over the items lives in LDS

// first key a query at position length - 1 may see (window_left < 0: no window)
ARENO_HD int first_visible_key(int length, int window_left) {
  if (window_left < 0) return 0;
  const int lo = length - 1 - window_left;
  return lo > 0 ? lo : 0;
}

struct UnitGeometry {
  int total_tiles;
  int units;
  bool narrow;  // the products below fit 32 bits: 32-bit divisions are a fifth of the instructions of 64-bit ones

  ARENO_HD int unit_start(int u) const {
    if (narrow)
      return static_cast<int>(static_cast<uint32_t>(u) * static_cast<uint32_t>(total_tiles) /
                              static_cast<uint32_t>(units));
    return static_cast<int>(static_cast<long long>(u) * total_tiles / units);
  }
  // unit that owns tile x, 0 <= x < total_tiles: the largest u with unit_start(u) <= x
  ARENO_HD int unit_of(int x) const {
    if (narrow)
      return static_cast<int>((static_cast<uint32_t>(x + 1) * static_cast<uint32_t>(units) +
                               static_cast<uint32_t>(total_tiles) - 1u) /
                              static_cast<uint32_t>(total_tiles)) -
             1;
    return static_cast<int>((static_cast<long long>(x + 1) * units + total_tiles - 1) / total_tiles - 1);
  }
};

ARENO_HD UnitGeometry make_unit_geometry(int total_tiles, int units) {
  UnitGeometry g;
  g.total_tiles = total_tiles;
  g.units = units;
  // largest product in unit_start / unit_of: (total_tiles + 1) * units + total_tiles
  g.narrow = (static_cast<long long>(total_tiles) + 2) * (static_cast<long long>(units) + 1) < (1LL << 31);
  return g;
}

// How the rows of a launch become items.
struct ItemShape {
  int batch;
  int window_left;
  int new_token_tile;  // 1: per-row items end in a tile of their own for the token being appended
  // prefix groups; num_shared = 0 and the other three = 1 without them
  int num_shared;      // shared items, listed in front of the per-row items
  int group_rows;      // rows per prefix group
  int cols_seqs;       // rows that fit side by side: 16 / (q heads per kv head)
  int subs_per_group;  // ceil(group_rows / cols_seqs)

  ARENO_HD int num_items() const { return num_shared + batch; }
  ARENO_HD int num_groups() const { return group_rows > 0 ? batch / group_rows : 0; }
};

struct ItemInfo {
  int lo;       // first token
  int end;      // end of the cached tokens the item reads through the block table of `row`
  int row;      // block-table / query row (first row of the sub-group for a shared item)
  int nseq;     // rows served side by side (1 for a per-row item)
  int has_new;  // a tile for the newest token follows the cached ones
  ARENO_HD int tiles() const { return (end - lo + kTileTokens - 1) / kTileTokens + has_new; }
};

// Lens supplies  int row_len(int row)  (cache_seqlens)  and  int group_len(int group)  (shared_prefix_lens).
// Tokens of a sub-group's shared prefix: the caller's figure, clipped to what every member has cached and cut to a
// whole number of tiles.
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
  ItemInfo it = {0, 0, 0, 1, 0};
  if constexpr (GROUPED) {
    if (v < s.num_shared) {
      it.end = shared_prefix_tokens(s, lens, v, it.row, it.nseq);
      return it;
    }
    const int b = v - s.num_shared;
    const int gi = b / s.group_rows;
    int row0, count;
    it.lo = shared_prefix_tokens(s, lens, gi * s.subs_per_group + (b - gi * s.group_rows) / s.cols_seqs, row0, count);
    it.end = lens.row_len(b) + 1 - s.new_token_tile;
    it.row = b;
    it.has_new = s.new_token_tile;
    return it;
  } else {
    const int len = lens.row_len(v);
    it.lo = first_visible_key(len + 1, s.window_left);
    it.end = len + 1 - s.new_token_tile;
    it.row = v;
    it.has_new = s.new_token_tile;
    return it;
  }
}

// Position of a tile stream: item, first token of the tile, the global index of the item's last tile + 1.
struct TileCursor {
  int b;
  int tok;
  int x_end;  // cum[b + 1]
  ItemInfo it;
  // the tile holds only the token being appended (no cached tokens left in the item)
  ARENO_HD bool on_new_token() const { return tok >= it.end; }
};

// Cum supplies  int at(int i)  = tiles of items [0, i), 0 <= i <= num_items.
// Put the cursor on global tile x (0 <= x < cum.at(num_items)).
template <bool GROUPED, class Lens, class Cum>
ARENO_HD void cursor_seek(TileCursor& c, const ItemShape& s, const Lens& lens, const Cum& cum, int x) {
  int lo = 0, hi = s.num_items();
  while (lo + 1 < hi) {  // the largest item index with cum <= x; items without tiles in front of it are skipped
    const int mid = (lo + hi) >> 1;
    if (cum.at(mid) <= x) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  c.b = lo;
  c.it = item_info<GROUPED>(s, lens, lo);
  c.tok = c.it.lo + (x - cum.at(lo)) * kTileTokens;
  c.x_end = cum.at(lo + 1);
}

// Move the cursor from tile x_next - 1 to tile x_next (x_next < cum.at(num_items)); true when that tile opens an item.
template <bool GROUPED, class Lens, class Cum>
ARENO_HD bool cursor_advance(TileCursor& c, const ItemShape& s, const Lens& lens, const Cum& cum, int x_next) {
  if (x_next != c.x_end) {
    c.tok += kTileTokens;
    return false;
  }
  int b = c.b + 1;
  int end = cum.at(b + 1);
  while (end == x_next) {  // items without tiles (a group with no shared prefix); ends before num_items because
    ++b;                   // x_next is a tile of some item
    end = cum.at(b + 1);
  }
  c.b = b;
  c.x_end = end;
  c.it = item_info<GROUPED>(s, lens, b);
  c.tok = c.it.lo;
  return true;
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
