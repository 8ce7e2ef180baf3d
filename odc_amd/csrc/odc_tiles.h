// odc_tiles.h — how a launch of libodc_hip.so is cut into tiles, and how a tile finds its work.
//
// Shared by the kernels (device), by the launch code (host) and by the CPU geometry test, which
// compiles this header with g++ alone and checks, by brute force, that every unit of every rank
// segment is owned by exactly one tile role and that no role reaches outside its segment.
//
// Vocabulary. A launch carries up to kMaxItems ITEMS (one shard of one tensor). An item has one
// SEGMENT per rank: `n` units (bytes or elements) at the same symmetric offset of every rank
// region. A segment is cut into TILES of kTileVecs vectors; a 256-thread workgroup does one tile
// at a time.
#ifndef ODC_TILES_H_
#define ODC_TILES_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define ODC_HD __host__ __device__ __forceinline__
#else
#define ODC_HD inline
#endif

#ifndef ODC_TILE_THREADS
#define ODC_TILE_THREADS 256  // 4 wavefronts of 64 lanes
#endif
#ifndef ODC_TILE_UNROLL
#define ODC_TILE_UNROLL 4  // independent vector accesses per lane per stream before the stores
#endif
#ifndef ODC_BODY_ALIGN
#define ODC_BODY_ALIGN 128  // bytes: alignment of a segment's vector body on the written side
#endif
#ifndef ODC_MAX_ITEMS_PER_LAUNCH
#define ODC_MAX_ITEMS_PER_LAUNCH 64
#endif

namespace odc_tiles {

constexpr int kThreads = ODC_TILE_THREADS;
constexpr int kUnroll = ODC_TILE_UNROLL;
constexpr int kMaxItems = ODC_MAX_ITEMS_PER_LAUNCH;
constexpr uint32_t kTileVecs = kThreads * kUnroll;  // vectors per tile
constexpr uint32_t kTileBytes = kTileVecs * 16;     // gather / clear: 16 KiB of destination
constexpr uint32_t kTileElems = kTileVecs * 4;      // accumulate / cast / publish: 4096 elements
constexpr uint64_t kMaxTilesPerLaunch = 1ull << 31;

// Tile order of a launch (TileTable::order).
//   kRanksInterleaved : item by item; within an item tile c of rank 0, of rank 1, ..., then c+1
//   kItemMajor        : item by item; within an item all of rank 0's tiles, then rank 1's
//   kRankOutermost    : rank by rank; within a rank item by item
enum TileOrder : uint32_t { kRanksInterleaved = 0, kItemMajor = 1, kRankOutermost = 2 };

// Travels by value in the kernel-argument segment. seg_prefix[i] is the number of tiles that
// the items before item i have in ONE rank segment each, so item i has
// seg_prefix[i+1] - seg_prefix[i] tiles per rank segment and world times that in the launch.
// Entries past n_items hold tiles_per_rank, so a search never lands on them.
struct TileTable {
  uint32_t world;
  uint32_t n_items;
  uint32_t n_tiles;         // world * tiles_per_rank
  uint32_t order;           // TileOrder
  uint32_t first_rank;      // rotation of the rank walk (never changes the result)
  uint32_t tiles_per_rank;  // seg_prefix[n_items]
  uint32_t seg_prefix[kMaxItems + 1];
};

struct TileCoord {
  uint32_t item, rank, chunk;  // chunk: tile index within the rank segment
};

// Largest i with seg_prefix[i] <= x, for x < tiles_per_rank (seg_prefix[0] is 0 and the entries
// are strictly increasing over the real items: empty items are never listed).
ODC_HD uint32_t find_item(const TileTable& tt, uint32_t x) {
  uint32_t lo = 0, hi = tt.n_items;
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (tt.seg_prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

// A cursor remembers the run of consecutive tile indices [lo, hi) that share the item (and, in
// rank-outermost order, the rank) of the last tile located, so a workgroup that walks many tiles
// with a grid-stride loop searches only when it leaves that run. Use:
//     if (!cursor_holds(cur, t)) {
//       cursor_seek(tt, t, cur);            // the search: sets cur.item
//       desc = launch.item[cur.item];       // the caller's per-item record ...
//       cursor_enter(tt, cur);              // ... and the run's bounds: independent loads
//     }
//     TileCoord c = cursor_coord(tt, cur, t);
struct TileCursor {
  uint32_t lo = 1, hi = 0;  // empty
  uint32_t item = 0;
  uint32_t rank = 0;  // kRankOutermost only: the (unrotated) rank of the run
  uint32_t tps = 1;   // tiles per rank segment of the item
};

ODC_HD bool cursor_holds(const TileCursor& cur, uint32_t t) { return t >= cur.lo && t < cur.hi; }

ODC_HD void cursor_seek(const TileTable& tt, uint32_t t, TileCursor& cur) {
  if (tt.order == kRankOutermost) {
    cur.rank = t / tt.tiles_per_rank;
    cur.item = find_item(tt, t - cur.rank * tt.tiles_per_rank);
  } else {
    // item i owns tiles [seg_prefix[i] * world, seg_prefix[i+1] * world)
    cur.rank = 0;
    cur.item = find_item(tt, t / tt.world);
  }
}

ODC_HD void cursor_enter(const TileTable& tt, TileCursor& cur) {
  const uint32_t first = tt.seg_prefix[cur.item], next = tt.seg_prefix[cur.item + 1];
  cur.tps = next - first;
  if (tt.order == kRankOutermost) {
    cur.lo = cur.rank * tt.tiles_per_rank + first;
    cur.hi = cur.lo + cur.tps;
  } else {
    cur.lo = first * tt.world;
    cur.hi = next * tt.world;
  }
}

// Tile t (inside the cursor's run) -> (item, rank, chunk). Everything here is wave-uniform.
ODC_HD TileCoord cursor_coord(const TileTable& tt, const TileCursor& cur, uint32_t t) {
  TileCoord c;
  const uint32_t lt = t - cur.lo;
  c.item = cur.item;
  if (tt.order == kRankOutermost) {
    c.rank = cur.rank;
    c.chunk = lt;
  } else if (tt.order == kItemMajor) {
    c.rank = lt / cur.tps;
    c.chunk = lt - c.rank * cur.tps;
  } else {
    c.chunk = lt / tt.world;
    c.rank = lt - c.chunk * tt.world;
  }
  c.rank += tt.first_rank;
  if (c.rank >= tt.world) c.rank -= tt.world;
  return c;
}

// The three steps in one call. Returns true when the cursor moved to another run.
ODC_HD bool locate_tile(const TileTable& tt, uint32_t t, TileCursor& cur, TileCoord& c) {
  const bool moved = !cursor_holds(cur, t);
  if (moved) {
    cursor_seek(tt, t, cur);
    cursor_enter(tt, cur);
  }
  c = cursor_coord(tt, cur, t);
  return moved;
}

// Shape of one rank segment of `n` units whose WRITTEN side starts at address D:
//     head  : the units before the first 128-byte line boundary of D (at most 127 bytes),
//     body  : nvec whole vectors, written with aligned 128-bit (64-bit for 16-bit outputs) stores,
//     tail  : what is left after the last whole vector.
// Tile c owns body vectors [c*kTileVecs, (c+1)*kTileVecs); tile 0 also does the head, and the
// tile holding the last body vector (tile 0 when there is none) the tail. The READ side takes
// whatever misalignment that leaves it with: gfx950 global loads accept any address.
struct SegShape {
  uint32_t head;  // units before the first line boundary of the written side (clipped to the segment)
  uint32_t tail;  // units after the last whole vector
  uint64_t nvec;  // whole vectors
  uint64_t last;  // tile that owns the tail
};

// unit_bytes: size of one unit on the written side; vec_units: units per vector
ODC_HD SegShape seg_shape(uintptr_t written_addr, uint64_t n, uint32_t unit_bytes, uint32_t vec_units) {
  // The body starts on a 128 B line of the written side, not merely on a vector boundary: a
  // wavefront's 64 vector stores then cover whole lines, none shared with the next wavefront.
  // (The head is at most 127 bytes, i.e. fewer units than a workgroup has lanes.)
  constexpr uint32_t kLine = ODC_BODY_ALIGN;
  static_assert(kLine >= 16 && kLine - 1 <= kThreads, "one lane per head unit");
  SegShape g;
  uint64_t head = ((kLine - (uint32_t)(written_addr & (kLine - 1))) & (kLine - 1)) / unit_bytes;
  if (head > n) head = n;
  g.head = (uint32_t)head;
  g.nvec = (n - head) / vec_units;
  g.tail = (uint32_t)((n - head) - g.nvec * vec_units);
  g.last = g.nvec ? (g.nvec - 1) / kTileVecs : 0;
  return g;
}

// Number of tiles of a segment of n units when a tile is tile_units units. (Upper bound of what
// the shape needs: a head shifts the body by less than one vector line, never past the count.)
ODC_HD uint64_t tiles_for(uint64_t n, uint64_t tile_units) { return (n + tile_units - 1) / tile_units; }

// What tile `chunk` of a segment does.
struct TileWork {
  uint64_t v0;     // first body vector of the tile
  uint32_t nv;     // body vectors of the tile (0 .. kTileVecs)
  bool head, tail; // also does the segment's head / tail
};

ODC_HD TileWork tile_work(uint32_t chunk, const SegShape& g) {
  TileWork w;
  w.v0 = (uint64_t)chunk * kTileVecs;
  w.nv = w.v0 >= g.nvec ? 0u : (g.nvec - w.v0 >= kTileVecs ? kTileVecs : (uint32_t)(g.nvec - w.v0));
  w.head = chunk == 0 && g.head != 0;
  w.tail = chunk == g.last && g.tail != 0;
  return w;
}

// A tile is a whole run when all its kTileVecs vectors exist: the unrolled, unguarded loop.
ODC_HD bool is_whole(const TileWork& w) { return w.nv == kTileVecs; }
// True when the tile has anything else to do: a partial run, the head or the tail.
ODC_HD bool has_edges(const TileWork& w) { return (w.nv != 0 && w.nv != kTileVecs) || w.head || w.tail; }

// Cuts items [*next, n_items) into one launch: at most kMaxItems non-empty items and fewer than
// kMaxTilesPerLaunch tiles. units(i) is item i's per-rank size in tile units (0 = skip);
// take(slot, i) copies item i's descriptor into slot `slot` of the launch. Returns the number of
// items taken (0 when only empty items were left), or -1 - i when item i alone is too large for
// one launch.
template <class Units, class Take>
inline int fill_tile_table(TileTable& tt, uint32_t world, uint32_t n_items, uint32_t* next,
                           uint64_t tile_units, Units units, Take take) {
  uint32_t n = 0;
  uint64_t tiles = 0, per_rank = 0;
  uint32_t i = *next;
  for (; i < n_items && n < (uint32_t)kMaxItems; ++i) {
    const uint64_t sz = units(i);
    if (sz == 0) continue;
    const uint64_t tps = tiles_for(sz, tile_units);
    if (tps * world >= kMaxTilesPerLaunch) return -1 - (int)i;
    if (tiles + tps * world >= kMaxTilesPerLaunch) break;
    tt.seg_prefix[n] = (uint32_t)per_rank;
    take(n, i);
    tiles += tps * world;
    per_rank += tps;
    ++n;
  }
  *next = i;
  for (uint32_t k = n; k <= (uint32_t)kMaxItems; ++k) tt.seg_prefix[k] = (uint32_t)per_rank;
  tt.world = world;
  tt.n_items = n;
  tt.n_tiles = (uint32_t)tiles;
  tt.tiles_per_rank = (uint32_t)per_rank;
  return (int)n;
}

}  // namespace odc_tiles

#endif  // ODC_TILES_H_
