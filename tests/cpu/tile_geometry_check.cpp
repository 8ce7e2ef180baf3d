// CPU check of odc_amd/csrc/odc_tiles.h, the tile geometry the HIP kernels index memory with.
// Built by tests/test_tile_geometry.py with g++ -fsanitize=address,undefined; no GPU involved.
//
// For random and edge-case item lists it builds launches with fill_tile_table exactly as the
// library does, walks every tile the way the kernels do (one workgroup per tile, and persistent
// workgroups with a grid-stride loop and a cursor), and asserts that
//   * tile t maps to the (item, rank, chunk) that a plain enumeration of the order gives,
//   * every unit of every rank segment is owned by exactly one role (head, body, tail) of
//     exactly one tile, and no role reaches outside its segment,
//   * body vectors are aligned on the written side and the body starts on a 128-byte line.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "odc_tiles.h"

using namespace odc_tiles;

static long g_checks = 0;
#define REQUIRE(cond, ...)                                   \
  do {                                                       \
    ++g_checks;                                              \
    if (!(cond)) {                                           \
      std::printf("FAILED %s:%d: %s\n  ", __FILE__, __LINE__, #cond); \
      std::printf(__VA_ARGS__);                              \
      std::printf("\n");                                     \
      std::exit(1);                                          \
    }                                                        \
  } while (0)

struct Item {
  uint64_t n;        // units per rank segment
  uint64_t written;  // address of rank 0's written side
  uint64_t stride;   // distance between the written sides of consecutive ranks, in bytes
};

struct Kind {
  uint32_t unit_bytes, vec_units;
  uint64_t tile_units;
};
static const Kind kKinds[] = {
    {1, 16, kTileBytes},  // gather / clear: bytes, 16-byte vectors
    {4, 4, kTileElems},   // fp32 accumulations / outputs: 4 elements per 16-byte vector
    {2, 4, kTileElems},   // 16-bit accumulations / outputs: 4 elements per 8-byte vector
};

static uint32_t tiles_per_seg(const TileTable& tt, uint32_t i) { return tt.seg_prefix[i + 1] - tt.seg_prefix[i]; }

// The order's definition, enumerated the slow way: the sequence of (slot, unrotated rank, chunk).
static std::vector<TileCoord> enumerate_order(const TileTable& tt) {
  std::vector<TileCoord> seq;
  if (tt.order == kRankOutermost) {
    for (uint32_t r = 0; r < tt.world; ++r)
      for (uint32_t i = 0; i < tt.n_items; ++i)
        for (uint32_t c = 0; c < tiles_per_seg(tt, i); ++c) seq.push_back({i, r, c});
  } else if (tt.order == kItemMajor) {
    for (uint32_t i = 0; i < tt.n_items; ++i)
      for (uint32_t r = 0; r < tt.world; ++r)
        for (uint32_t c = 0; c < tiles_per_seg(tt, i); ++c) seq.push_back({i, r, c});
  } else {
    for (uint32_t i = 0; i < tt.n_items; ++i)
      for (uint32_t c = 0; c < tiles_per_seg(tt, i); ++c)
        for (uint32_t r = 0; r < tt.world; ++r) seq.push_back({i, r, c});
  }
  return seq;
}

static void check_launch(const TileTable& tt0, const std::vector<Item>& slots, const Kind& kind, std::mt19937_64& rng) {
  for (uint32_t order = 0; order < 3; ++order) {
    TileTable tt = tt0;
    tt.order = order;
    tt.first_rank = (uint32_t)(rng() % tt.world);
    const std::vector<TileCoord> want = enumerate_order(tt);
    REQUIRE(want.size() == tt.n_tiles, "order %u: %zu enumerated, n_tiles %u", order, want.size(), tt.n_tiles);
    // coverage counters per (slot, rank, unit)
    std::vector<std::vector<std::vector<uint8_t>>> seen(tt.n_items);
    for (uint32_t i = 0; i < tt.n_items; ++i) seen[i].assign(tt.world, std::vector<uint8_t>(slots[i].n, 0));
    // grid shapes: one workgroup per tile, and a few persistent grids
    const uint32_t grids[] = {tt.n_tiles, 1u, 7u, (uint32_t)(1 + rng() % 300)};
    for (int gsel = 0; gsel < 4; ++gsel) {
      const uint32_t grid = grids[gsel] < tt.n_tiles ? grids[gsel] : tt.n_tiles;
      for (uint32_t b = 0; b < grid; ++b) {
        TileCursor cur, cur2;
        uint32_t held_item = ~0u;
        for (uint32_t t = b; t < tt.n_tiles; t += grid) {
          // exactly the kernels' sequence
          if (!cursor_holds(cur, t)) {
            cursor_seek(tt, t, cur);
            held_item = cur.item;  // what a kernel reloads its descriptor for
            cursor_enter(tt, cur);
            REQUIRE(cursor_holds(cur, t), "t %u is outside the run the cursor entered", t);
          }
          const TileCoord c = cursor_coord(tt, cur, t);
          REQUIRE(held_item == c.item, "t %u: the cursor changed item without saying so", t);
          TileCoord c2;
          locate_tile(tt, t, cur2, c2);
          REQUIRE(c2.item == c.item && c2.rank == c.rank && c2.chunk == c.chunk, "locate_tile disagrees at t %u", t);
          const uint32_t rot = (want[t].rank + tt.first_rank) % tt.world;
          REQUIRE(c.item == want[t].item && c.rank == rot && c.chunk == want[t].chunk,
                  "order %u first_rank %u grid %u t %u: got (%u,%u,%u) want (%u,%u,%u)", order, tt.first_rank, grid,
                  t, c.item, c.rank, c.chunk, want[t].item, rot, want[t].chunk);
          if (gsel != 0) continue;  // coverage is counted once, on the one-workgroup-per-tile walk
          const Item& it = slots[c.item];
          const uint64_t addr = it.written + (uint64_t)c.rank * it.stride;
          const SegShape g = seg_shape((uintptr_t)addr, it.n, kind.unit_bytes, kind.vec_units);
          REQUIRE((uint64_t)g.head + g.nvec * kind.vec_units + g.tail == it.n, "shape does not add up: n %llu",
                  (unsigned long long)it.n);
          REQUIRE(g.tail < kind.vec_units && g.head * kind.unit_bytes < ODC_BODY_ALIGN, "head %u tail %u", g.head, g.tail);
          REQUIRE(g.head <= (uint32_t)kThreads && g.tail <= (uint32_t)kThreads, "one lane per head/tail unit");
          const TileWork w = tile_work(c.chunk, g);
          REQUIRE(is_whole(w) == (w.nv == kTileVecs), "is_whole");
          REQUIRE(has_edges(w) == ((w.nv != 0 && w.nv != kTileVecs) || w.head || w.tail), "has_edges");
          std::vector<uint8_t>& u = seen[c.item][c.rank];
          auto mark = [&](uint64_t lo, uint64_t hi, const char* role) {
            REQUIRE(hi <= it.n, "%s [%llu, %llu) leaves a segment of %llu units (chunk %u)", role,
                    (unsigned long long)lo, (unsigned long long)hi, (unsigned long long)it.n, c.chunk);
            for (uint64_t k = lo; k < hi; ++k) u[k]++;
          };
          if (w.head) mark(0, g.head, "head");
          if (w.nv) {
            REQUIRE(w.v0 + w.nv <= g.nvec, "body past nvec");
            const uint64_t e0 = g.head + w.v0 * kind.vec_units;
            const uint64_t body_addr = addr + e0 * kind.unit_bytes;
            REQUIRE(body_addr % (kind.vec_units * kind.unit_bytes) == 0, "body vector misaligned");
            if (w.v0 == 0 && g.head) REQUIRE(body_addr % ODC_BODY_ALIGN == 0, "body does not start on a line");
            mark(e0, e0 + (uint64_t)w.nv * kind.vec_units, "body");
          }
          if (w.tail) mark(g.head + g.nvec * kind.vec_units, it.n, "tail");
        }
      }
    }
    for (uint32_t i = 0; i < tt.n_items; ++i)
      for (uint32_t r = 0; r < tt.world; ++r)
        for (uint64_t k = 0; k < slots[i].n; ++k)
          REQUIRE(seen[i][r][k] == 1, "order %u slot %u rank %u unit %llu of %llu owned %u times", order, i, r,
                  (unsigned long long)k, (unsigned long long)slots[i].n, seen[i][r][k]);
  }
}

static uint64_t pick_size(std::mt19937_64& rng, uint64_t tile_units) {
  static const uint64_t edge[] = {0, 1, 15, 16, 17, 127, 128, 129, 255, 256, 4095, 4096, 4097, 16383, 16384, 16385};
  switch (rng() % 5) {
    case 0: return edge[rng() % (sizeof(edge) / sizeof(edge[0]))];
    case 1: return tile_units * (1 + rng() % 3) + (rng() % 3) - 1;  // k * tile +- 1
    case 2: return rng() % 200;
    case 3: return rng() % (3 * tile_units);
    default: return 64 * (rng() % 100);
  }
}

static void run_case(std::mt19937_64& rng, uint32_t world, uint32_t n_items, const Kind& kind) {
  std::vector<Item> items(n_items);
  for (Item& it : items) {
    it.n = pick_size(rng, kind.tile_units);
    const uint64_t align = (rng() % 3 == 0) ? 256 : kind.unit_bytes;  // arena offsets are 256 B aligned
    it.written = (1ull << 40) + (rng() % 4096) / align * align;
    // gather: consecutive blocks of the output; accumulate: one offset in every rank region
    it.stride = (rng() & 1) ? it.n * kind.unit_bytes : (1ull << 30) + 256 * (rng() % 8);
  }
  uint32_t next = 0, launches = 0;
  while (next < n_items) {
    TileTable tt;
    std::vector<Item> slots;
    const int n = fill_tile_table(
        tt, world, n_items, &next, kind.tile_units, [&](uint32_t i) { return items[i].n; },
        [&](uint32_t slot, uint32_t i) {
          REQUIRE(slot == slots.size() && slot < (uint32_t)kMaxItems, "slot %u", slot);
          slots.push_back(items[i]);
        });
    REQUIRE(n >= 0 && n <= kMaxItems, "fill_tile_table returned %d", n);
    if (n == 0) continue;
    ++launches;
    REQUIRE(tt.n_items == (uint32_t)n && tt.world == world && tt.tiles_per_rank * world == tt.n_tiles, "table header");
    REQUIRE(tt.seg_prefix[0] == 0, "prefix starts at 0");
    for (uint32_t k = 0; k < tt.n_items; ++k)
      REQUIRE(tiles_per_seg(tt, k) == tiles_for(slots[k].n, kind.tile_units) && tiles_per_seg(tt, k) > 0, "prefix %u", k);
    for (uint32_t k = tt.n_items; k <= (uint32_t)kMaxItems; ++k)
      REQUIRE(tt.seg_prefix[k] == tt.tiles_per_rank, "padding %u", k);
    check_launch(tt, slots, kind, rng);
  }
  uint32_t nonempty = 0;
  for (const Item& it : items) nonempty += it.n != 0;
  REQUIRE(launches == (nonempty + kMaxItems - 1) / kMaxItems, "%u launches for %u non-empty items", launches, nonempty);
}

int main(int argc, char** argv) {
  const uint64_t seed = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 1;
  const int cases = argc > 2 ? std::atoi(argv[2]) : 400;
  std::mt19937_64 rng(seed);
  // every world size 1..200 at least once with a short list, plus random cases
  for (uint32_t world = 1; world <= 200; ++world) run_case(rng, world, 1 + rng() % 4, kKinds[world % 3]);
  for (int k = 0; k < cases; ++k) {
    const uint32_t world = 1 + (uint32_t)(rng() % (k % 7 == 0 ? 200 : 16));
    const uint32_t n_items = (k % 23 == 0) ? 65 + (uint32_t)(rng() % 80) : 1 + (uint32_t)(rng() % 20);
    run_case(rng, world, world > 32 && n_items > 64 ? 66 : n_items, kKinds[rng() % 3]);
  }
  // an item too large for one launch is refused, not truncated
  {
    TileTable tt;
    uint32_t next = 0;
    const int n = fill_tile_table(
        tt, 8, 1, &next, kTileElems, [&](uint32_t) { return (uint64_t)kTileElems * (kMaxTilesPerLaunch / 8); },
        [&](uint32_t, uint32_t) {});
    REQUIRE(n == -1, "oversized item: %d", n);
  }
  std::printf("tile geometry ok: %ld checks\n", g_checks);
  return 0;
}
