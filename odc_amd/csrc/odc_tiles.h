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

// Travels by value in the kernel-argument segment. Item i owns tiles
// [tile_prefix[i], tile_prefix[i+1]) (in the item-major orders), which are
// world * tiles_per_seg[i] tiles: one run of tiles_per_seg[i] per rank segment. Entries past
// n_items hold n_tiles, so a search never lands on them.
struct TileTable {
  uint32_t world;
  uint32_t n_items;
  uint32_t n_tiles;
  uint32_t order;           // TileOrder
  uint32_t first_rank;      // rotation of the rank walk (never changes the result)
  uint32_t tiles_per_rank;  // n_tiles / world
  uint32_t tile_prefix[kMaxItems + 1];
  uint32_t tiles_per_seg[kMaxItems];
};

struct TileCoord {
  uint32_t item, rank, chunk;  // chunk: tile index within the rank segment
};

// Largest i with tile_prefix[i] <= x, for x < n_tiles (tile_prefix[0] is 0 and the entries are
// strictly increasing over the real items: empty items are never listed).
ODC_HD uint32_t find_item(const TileTable& tt, uint64_t x) {
  uint32_t lo = 0, hi = tt.n_items;
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (tt.tile_prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

// A cursor remembers the run of consecutive tile indices [lo, hi) that share the item (and, in
// rank-outermost order, the rank) of the last tile located, so a workgroup that walks many tiles
// with a grid-stride loop searches only when it leaves that run.
struct TileCursor {
  uint32_t lo = 1, hi = 0;  // empty
  uint32_t item = 0;
  uint32_t rank = 0;  // kRankOutermost only: the (unrotated) rank of the run
  uint32_t tps = 1;   // tiles_per_seg[item]
};

// Tile t of a launch -> (item, rank, chunk). Returns true when the cursor moved to another item
// (the caller then reloads the item's descriptor). Everything here is wave-uniform.
ODC_HD bool locate_tile(const TileTable& tt, uint32_t t, TileCursor& cur, TileCoord& c) {
  bool moved = false;
  if (t < cur.lo || t >= cur.hi) {
    moved = true;
    if (tt.order == kRankOutermost) {
      // tile_prefix[i] is world times the tiles before item i within one rank
      const uint32_t rank = t / tt.tiles_per_rank;
      const uint32_t local = t - rank * tt.tiles_per_rank;
      const uint32_t i = find_item(tt, (uint64_t)local * tt.world);
      cur.item = i;
      cur.rank = rank;
      cur.tps = tt.tiles_per_seg[i];
      cur.lo = rank * tt.tiles_per_rank + tt.tile_prefix[i] / tt.world;
      cur.hi = cur.lo + cur.tps;
    } else {
      const uint32_t i = find_item(tt, t);
      cur.item = i;
      cur.tps = tt.tiles_per_seg[i];
      cur.lo = tt.tile_prefix[i];
      cur.hi = tt.tile_prefix[i + 1];
    }
  }
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
  uint64_t tiles = 0;
  uint32_t i = *next;
  for (; i < n_items && n < (uint32_t)kMaxItems; ++i) {
    const uint64_t sz = units(i);
    if (sz == 0) continue;
    const uint64_t tps = tiles_for(sz, tile_units);
    if (tps * world >= kMaxTilesPerLaunch) return -1 - (int)i;
    if (tiles + tps * world >= kMaxTilesPerLaunch) break;
    tt.tile_prefix[n] = (uint32_t)tiles;
    tt.tiles_per_seg[n] = (uint32_t)tps;
    take(n, i);
    tiles += tps * world;
    ++n;
  }
  *next = i;
  for (uint32_t k = n; k <= (uint32_t)kMaxItems; ++k) tt.tile_prefix[k] = (uint32_t)tiles;
  for (uint32_t k = n; k < (uint32_t)kMaxItems; ++k) tt.tiles_per_seg[k] = 1;
  tt.world = world;
  tt.n_items = n;
  tt.n_tiles = (uint32_t)tiles;
  tt.tiles_per_rank = world ? (uint32_t)(tiles / world) : 0;
  return (int)n;
}

}  // namespace odc_tiles

#endif  // ODC_TILES_H_
