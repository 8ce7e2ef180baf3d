// odc_host.cpp — the host side of libodc_hip.so: the C ABI of include/odc_hip.h, the symmetric
// arena (one device allocation, W rank regions, one offset valid in all), argument validation and
// launch planning. Plain C++: everything that needs the HIP runtime or a kernel is behind
// namespace odc_device (odc_launch.h), implemented for gfx950 in odc_kernels.hip. Built with g++
// against an odc_device that has no device, this file runs under AddressSanitizer and UBSan on
// bookkeeping-only and dry-run arenas.
//
// Launch model: the work of one launch is cut into tiles of 1024 vectors (16 KiB, odc_tiles.h);
// per-item descriptors (<= ODC_MAX_ITEMS_PER_LAUNCH) travel BY VALUE in the kernel argument
// segment, so a call needs no device-side work list, no host->device copy and no allocation;
// longer item lists are split over several launches.

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "odc_hip.h"
#include "odc_launch.h"
#include "odc_tiles.h"

namespace {

// ------------------------------------------------------------------------------------------------
// errors
// ------------------------------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define ODC_DEVICE_TRY(expr)                                                                   \
  do {                                                                                         \
    const int e_ = (expr);                                                                     \
    if (e_ != 0)                                                                               \
      return fail(ODC_ERR_HIP, "%s failed: %s (%s:%d)", #expr, odc_device::error_string(e_),   \
                  __FILE__, __LINE__);                                                         \
  } while (0)

// ------------------------------------------------------------------------------------------------
// options
// ------------------------------------------------------------------------------------------------
struct Options {
  // measured on MI355X over a Llama-3-8B layer: every kernel peaks with one workgroup per tile
  // and no residency cap
  int64_t gather_blocks_per_cu = 0;
  int64_t gather_resident_cap = 0;  // 512-thread workgroups: 4 per CU without a cap
  int64_t cast_resident_cap = 0;
  int64_t accum_resident_cap = 0;
  int64_t accum_blocks_per_cu = -1;  // -1: by segment length (see scatter_launch)
  int64_t accum_short_segment_tiles = 256;   // segments averaging fewer tiles: rank-outermost tile order
  int64_t accum_persistent_below_tiles = 0;  // segments averaging fewer tiles: persistent launch shape (0: never)
  int64_t accum_small_items_last = 1;  // scatter launches: items of less than one tile per rank go last
  int64_t store_blocks_per_cu = 0;  // the scatter-store (no read of the accumulation)
  int64_t store_resident_cap = 0;  // 512-thread workgroups, like the gathers
  int64_t clear_blocks_per_cu = 0;
  int64_t publish_blocks_per_cu = 0;
  int64_t publish_resident_cap = 0;
  int64_t rank_major = 1;        // gather: 0 = ranks interleaved, 1 = item-major, 2 = rank outermost
  int64_t accum_tile_order = 3;  // the same for scatter-accumulate / store; 3 = by segment length
  int64_t rank_stagger_bytes = 0;
  int64_t rank_stride_align = 16384;  // rank regions start on multiples of this (read when an arena is created)
  int64_t alloc_align = 16384;        // so do symmetric allocations at least this large
};
Options g_opt;
std::mutex g_opt_mu;

int64_t* option_slot(const char* name) {
  if (!name) return nullptr;
  if (!strcmp(name, "gather_blocks_per_cu")) return &g_opt.gather_blocks_per_cu;
  if (!strcmp(name, "accum_blocks_per_cu")) return &g_opt.accum_blocks_per_cu;
  if (!strcmp(name, "accum_short_segment_tiles")) return &g_opt.accum_short_segment_tiles;
  if (!strcmp(name, "accum_persistent_below_tiles")) return &g_opt.accum_persistent_below_tiles;
  if (!strcmp(name, "accum_small_items_last")) return &g_opt.accum_small_items_last;
  if (!strcmp(name, "clear_blocks_per_cu")) return &g_opt.clear_blocks_per_cu;
  if (!strcmp(name, "publish_blocks_per_cu")) return &g_opt.publish_blocks_per_cu;
  if (!strcmp(name, "rank_major")) return &g_opt.rank_major;
  if (!strcmp(name, "accum_tile_order")) return &g_opt.accum_tile_order;
  if (!strcmp(name, "rank_stagger_bytes")) return &g_opt.rank_stagger_bytes;
  if (!strcmp(name, "rank_stride_align")) return &g_opt.rank_stride_align;
  if (!strcmp(name, "alloc_align")) return &g_opt.alloc_align;
  if (!strcmp(name, "gather_resident_cap")) return &g_opt.gather_resident_cap;
  if (!strcmp(name, "cast_resident_cap")) return &g_opt.cast_resident_cap;
  if (!strcmp(name, "accum_resident_cap")) return &g_opt.accum_resident_cap;
  if (!strcmp(name, "store_blocks_per_cu")) return &g_opt.store_blocks_per_cu;
  if (!strcmp(name, "store_resident_cap")) return &g_opt.store_resident_cap;
  if (!strcmp(name, "publish_resident_cap")) return &g_opt.publish_resident_cap;
  return nullptr;
}

using namespace odc_tiles;
using namespace odc_launch;

// ------------------------------------------------------------------------------------------------
// host side: arena
// ------------------------------------------------------------------------------------------------
constexpr uint64_t kAlign = 256;

inline uint64_t round_up(uint64_t x, uint64_t a) { return (x + a - 1) / a * a; }

}  // namespace

struct odc_arena {
  uint32_t world = 0;
  int device = -1;
  uint32_t flags = 0;
  int n_cu = 256;
  int lds_per_cu = 160 * 1024;
  int lds_per_wg_max = 64 * 1024;
  uint64_t bytes_per_rank = 0;
  uint64_t rank_stride = 0;
  uint64_t alloc_align = 16384;
  void* allocation = nullptr;  // the one device allocation (null without backing)
  uint8_t* base = nullptr;    // rank 0's region: the allocation rounded up to the stride alignment
  uint8_t* origin = nullptr;  // what launches are planned against: base, or a fictitious address on a dry-run arena
  bool dry_run = false;
  std::map<uint64_t, uint64_t> live;  // offset -> size (rounded)
  std::map<uint64_t, uint64_t> free_; // offset -> size, coalesced
  uint64_t in_use = 0;
  uint64_t high_water = 0;
  std::mutex mu;
};

namespace {

int check_arena(const odc_arena* a) {
  if (!a) return fail(ODC_ERR_INVALID, "arena is NULL");
  return ODC_OK;
}

// Makes the arena's device current for the scope of one entry point and puts the caller's
// device back afterwards (the caller may be any host thread with any current device).
class DeviceGuard {
 public:
  DeviceGuard() = default;
  DeviceGuard(const DeviceGuard&) = delete;
  DeviceGuard& operator=(const DeviceGuard&) = delete;
  int enter(int device) {
    ODC_DEVICE_TRY(odc_device::get_current(&prev_));
    if (prev_ != device) {
      ODC_DEVICE_TRY(odc_device::set_current(device));
      switched_ = true;
    }
    return ODC_OK;
  }
  ~DeviceGuard() {
    if (switched_) (void)odc_device::set_current(prev_);
  }

 private:
  int prev_ = -1;
  bool switched_ = false;
};

int check_compute(odc_arena* a, DeviceGuard& guard) {
  if (int rc = check_arena(a)) return rc;
  if (a->dry_run) return ODC_OK;  // plans against a fictitious address, launches nothing
  if (!a->base)
    return fail(ODC_ERR_NO_BACKING, "arena has no device memory (created with ODC_ARENA_NO_BACKING)");
  return guard.enter(a->device);
}

// What dry-run arenas have "launched" (process-wide, reset by odc_set_option("dry_run_reset", 0)).
std::atomic<int64_t> g_dry_launches{0}, g_dry_tiles{0}, g_dry_workgroups{0};

// The one place kernels are launched from: `issue` is the odc_device launch of the entry point.
// On a dry-run arena the launch is only counted: the host-side validation, work-list splitting
// and tile tables have all run by then.
template <class Launch, class Issue>
int launch_tiles(const odc_arena* a, const Launch& L, uint32_t grid, Issue issue) {
  if (grid == 0 || grid > L.tt.n_tiles || L.tt.n_tiles != L.tt.tiles_per_rank * L.tt.world)
    return fail(ODC_ERR_INVALID, "internal: launch of %u workgroups over %u tiles", grid, L.tt.n_tiles);
  if (a->dry_run) {
    g_dry_launches += 1;
    g_dry_tiles += L.tt.n_tiles;
    g_dry_workgroups += grid;
    return ODC_OK;
  }
  const int e = issue();
  if (e != 0) return fail(ODC_ERR_HIP, "kernel launch failed: %s", odc_device::error_string(e));
  return ODC_OK;
}

Options options_snapshot() {
  std::lock_guard<std::mutex> lk(g_opt_mu);
  return g_opt;
}

// blocks_per_cu > 0 asks for that many persistent workgroups per CU. Ragged launches (uneven
// shards: unaligned reads, heads and tails) never get them: they hide their extra latency better
// with one workgroup per tile, i.e. full occupancy (measured: +5..10 %).
uint32_t grid_for(const odc_arena* a, int64_t blocks_per_cu, uint32_t n_tiles, bool ragged = false) {
  if (blocks_per_cu <= 0 || ragged) return n_tiles;
  const uint64_t g = (uint64_t)a->n_cu * (uint64_t)blocks_per_cu;
  return (uint32_t)std::min<uint64_t>(g, n_tiles);
}

// One-workgroup-per-tile launches are dealt out by the hardware dispatcher, which keeps as many
// workgroups resident as fit. Fewer resident workgroups (a smaller window of memory in flight)
// can stream faster; the only lever is to make each workgroup claim a share of the CU's LDS that
// it never touches. Returns the dynamic LDS bytes that leave room for exactly `cap` workgroups.
uint32_t lds_claim_for(const odc_arena* a, int64_t cap, uint32_t grid, uint32_t n_tiles) {
  if (cap <= 0 || grid != n_tiles) return 0;  // persistent grids size themselves
  const uint64_t per_wg = ((uint64_t)a->lds_per_cu / (uint64_t)cap) & ~(uint64_t)1023;
  return (uint32_t)std::min<uint64_t>(per_wg, (uint64_t)a->lds_per_wg_max);
}

}  // namespace

extern "C" {

const char* odc_last_error(void) { return g_err; }

int odc_abi_version(void) { return ODC_HIP_ABI_VERSION; }

int odc_set_option(const char* name, int64_t value) {
  if (name && !strcmp(name, "dry_run_reset")) {
    g_dry_launches = 0; g_dry_tiles = 0; g_dry_workgroups = 0;
    return ODC_OK;
  }
  std::lock_guard<std::mutex> lk(g_opt_mu);
  int64_t* s = option_slot(name);
  if (!s) return fail(ODC_ERR_INVALID, "unknown option '%s'", name ? name : "(null)");
  const bool may_be_auto = s == &g_opt.accum_blocks_per_cu;  // -1: chosen per launch
  if (value < (may_be_auto ? -1 : 0)) return fail(ODC_ERR_INVALID, "option '%s' must be >= 0", name);
  // the arena layout options enter address arithmetic: keep them where it cannot wrap around
  const bool is_layout = s == &g_opt.rank_stagger_bytes || s == &g_opt.rank_stride_align || s == &g_opt.alloc_align;
  if (is_layout && value > (int64_t(1) << 40))
    return fail(ODC_ERR_INVALID, "option '%s' must be <= 2^40", name);
  *s = value;
  return ODC_OK;
}

int odc_get_option(const char* name, int64_t* value) {
  if (name && value) {
    if (!strcmp(name, "dry_run_launches")) { *value = g_dry_launches.load(); return ODC_OK; }
    if (!strcmp(name, "dry_run_tiles")) { *value = g_dry_tiles.load(); return ODC_OK; }
    if (!strcmp(name, "dry_run_workgroups")) { *value = g_dry_workgroups.load(); return ODC_OK; }
  }
  std::lock_guard<std::mutex> lk(g_opt_mu);
  int64_t* s = option_slot(name);
  if (!s || !value) return fail(ODC_ERR_INVALID, "unknown option '%s'", name ? name : "(null)");
  *value = *s;
  return ODC_OK;
}

int odc_arena_create(uint32_t world_size, uint64_t bytes_per_rank, uint32_t flags,
                     odc_arena** out) {
  if (!out) return fail(ODC_ERR_INVALID, "out is NULL");
  *out = nullptr;
  if (world_size == 0) return fail(ODC_ERR_INVALID, "world_size must be >= 1");
  if (bytes_per_rank == 0) return fail(ODC_ERR_INVALID, "bytes_per_rank must be > 0");
  if (bytes_per_rank > (uint64_t(1) << 60)) return fail(ODC_ERR_INVALID, "bytes_per_rank must be <= 2^60");
  if (flags & ~(uint32_t)(ODC_ARENA_NO_BACKING | ODC_ARENA_DRY_RUN))
    return fail(ODC_ERR_INVALID, "unknown flags 0x%x", flags);
  if (flags & ODC_ARENA_DRY_RUN) flags |= ODC_ARENA_NO_BACKING;  // a dry run never owns device memory
  odc_arena* a = new (std::nothrow) odc_arena();
  if (!a) return fail(ODC_ERR_NOMEM, "host allocation failed");
  a->world = world_size;
  a->flags = flags;
  const Options opt = options_snapshot();
  const uint64_t stride_align = std::max<uint64_t>(round_up((uint64_t)opt.rank_stride_align, kAlign), kAlign);
  a->alloc_align = std::max<uint64_t>(round_up((uint64_t)opt.alloc_align, kAlign), kAlign);
  a->bytes_per_rank = round_up(bytes_per_rank, kAlign);
  a->rank_stride = round_up(a->bytes_per_rank + round_up((uint64_t)opt.rank_stagger_bytes, kAlign), stride_align);
  // the device allocation promises 256 B alignment only; the regions shall start on stride_align
  // boundaries, so the allocation is that much larger: the whole sum must fit 64 bits
  const uint64_t slack = stride_align > kAlign ? stride_align : 0;
  if (a->rank_stride > (~0ull - slack) / world_size) {
    delete a;
    return fail(ODC_ERR_INVALID, "arena size overflows 64 bits");
  }
  if (!(flags & ODC_ARENA_NO_BACKING)) {
    odc_device::Properties prop = {};
    int e = odc_device::get_current(&a->device);
    if (e == 0) e = odc_device::properties(a->device, &prop);
    void* p = nullptr;
    if (e == 0) e = odc_device::allocate(&p, a->rank_stride * world_size + slack);
    if (e != 0) {
      delete a;
      return fail(odc_device::is_out_of_memory(e) ? ODC_ERR_NOMEM : ODC_ERR_HIP,
                  "creating a %u x %llu byte arena failed: %s", world_size,
                  (unsigned long long)bytes_per_rank, odc_device::error_string(e));
    }
    a->n_cu = prop.n_cu;
    a->lds_per_cu = prop.lds_per_cu;
    a->lds_per_wg_max = prop.lds_per_wg_max;
    a->allocation = p;
    a->base = reinterpret_cast<uint8_t*>(round_up((uint64_t)(uintptr_t)p, stride_align));
    a->origin = a->base;
  } else if (flags & ODC_ARENA_DRY_RUN) {
    a->dry_run = true;
    a->origin = reinterpret_cast<uint8_t*>(uintptr_t(1) << 44);  // never dereferenced
  }
  a->free_[0] = a->bytes_per_rank;
  *out = a;
  return ODC_OK;
}

int odc_arena_destroy(odc_arena* a) {
  if (int rc = check_arena(a)) return rc;
  int rc = ODC_OK;
  if (a->base) {
    int cur = -1;
    int e = odc_device::get_current(&cur);
    if (e == 0 && cur != a->device) e = odc_device::set_current(a->device);
    if (e == 0) e = odc_device::release(a->allocation);
    if (e != 0) rc = fail(ODC_ERR_HIP, "releasing the arena failed: %s", odc_device::error_string(e));
  }
  delete a;
  return rc;
}

int odc_arena_alloc(odc_arena* a, uint64_t nbytes, uint64_t* offset) {
  if (int rc = check_arena(a)) return rc;
  if (!offset) return fail(ODC_ERR_INVALID, "offset is NULL");
  std::lock_guard<std::mutex> lk(a->mu);
  const uint64_t need = std::max<uint64_t>(round_up(nbytes, kAlign), kAlign);
  if (need < nbytes) return fail(ODC_ERR_INVALID, "nbytes overflows");
  // a buffer of at least one tile starts on a tile-sized boundary (the read-modify-write of the
  // scatter-accumulate is up to 5.5 % slower on accumulations whose tiles straddle them);
  // smaller ones only need the 256 bytes the vector accesses want
  const uint64_t align = need >= a->alloc_align ? a->alloc_align : kAlign;
  for (auto it = a->free_.begin(); it != a->free_.end(); ++it) {  // first fit
    const uint64_t blk = it->first, blk_sz = it->second;
    const uint64_t off = round_up(blk, align);
    if (off < blk || off - blk > blk_sz || blk_sz - (off - blk) < need) continue;
    a->free_.erase(it);
    if (off > blk) a->free_[blk] = off - blk;  // the gap in front stays free
    if (blk + blk_sz > off + need) a->free_[off + need] = blk + blk_sz - (off + need);
    a->live[off] = need;
    a->in_use += need;
    a->high_water = std::max(a->high_water, off + need);
    *offset = off;
    return ODC_OK;
  }
  uint64_t largest = 0;
  for (const auto& blk : a->free_) largest = std::max(largest, blk.second);
  return fail(ODC_ERR_NOMEM,
              "symmetric arena exhausted: need %llu bytes per rank on a %llu-byte boundary, %llu of %llu "
              "in use, largest free block %llu (raise ODC_SYMMETRIC_SIZE)",
              (unsigned long long)need, (unsigned long long)align, (unsigned long long)a->in_use,
              (unsigned long long)a->bytes_per_rank, (unsigned long long)largest);
}

int odc_arena_free(odc_arena* a, uint64_t offset) {
  if (int rc = check_arena(a)) return rc;
  std::lock_guard<std::mutex> lk(a->mu);
  auto it = a->live.find(offset);
  if (it == a->live.end())
    return fail(ODC_ERR_NOT_FOUND, "offset %llu is not a live allocation", (unsigned long long)offset);
  uint64_t off = it->first, sz = it->second;
  a->live.erase(it);
  a->in_use -= sz;
  auto next = a->free_.lower_bound(off);
  if (next != a->free_.end() && off + sz == next->first) {  // merge with the block after
    sz += next->second;
    next = a->free_.erase(next);
  }
  if (next != a->free_.begin()) {  // merge with the block before
    auto prev = std::prev(next);
    if (prev->first + prev->second == off) {
      prev->second += sz;
      return ODC_OK;
    }
  }
  a->free_[off] = sz;
  return ODC_OK;
}

int odc_arena_reset(odc_arena* a) {
  if (int rc = check_arena(a)) return rc;
  std::lock_guard<std::mutex> lk(a->mu);
  a->live.clear();
  a->free_.clear();
  a->free_[0] = a->bytes_per_rank;
  a->in_use = 0;
  return ODC_OK;
}

int odc_arena_get_info(const odc_arena* a, odc_arena_info* info) {
  if (int rc = check_arena(a)) return rc;
  if (!info) return fail(ODC_ERR_INVALID, "info is NULL");
  odc_arena* m = const_cast<odc_arena*>(a);
  std::lock_guard<std::mutex> lk(m->mu);
  info->world_size = a->world;
  info->device = a->base ? a->device : -1;
  info->flags = a->flags;
  info->n_allocations = (uint32_t)a->live.size();
  info->bytes_per_rank = a->bytes_per_rank;
  info->rank_stride = a->rank_stride;
  info->base = (uint64_t)(uintptr_t)a->base;
  info->bytes_in_use = a->in_use;
  info->high_water = a->high_water;
  return ODC_OK;
}

void* odc_arena_ptr(const odc_arena* a, uint32_t rank, uint64_t offset) {
  if (!a || !a->base || rank >= a->world || offset > a->bytes_per_rank) {
    fail(ODC_ERR_INVALID, "odc_arena_ptr: bad arena, rank %u or offset %llu", rank,
         (unsigned long long)offset);
    return nullptr;
  }
  return a->base + (uint64_t)rank * a->rank_stride + offset;
}

int odc_arena_locate(const odc_arena* a, const void* ptr, uint32_t* rank, uint64_t* alloc_offset,
                     uint64_t* inner) {
  if (int rc = check_arena(a)) return rc;
  if (!a->base) return fail(ODC_ERR_NO_BACKING, "arena has no device memory");
  const uint8_t* p = static_cast<const uint8_t*>(ptr);
  if (p < a->base || p >= a->base + a->rank_stride * a->world)
    return fail(ODC_ERR_NOT_FOUND, "pointer %p is outside the arena", ptr);
  const uint64_t d = (uint64_t)(p - a->base);
  const uint32_t r = (uint32_t)(d / a->rank_stride);
  const uint64_t off = d - (uint64_t)r * a->rank_stride;
  odc_arena* m = const_cast<odc_arena*>(a);
  std::lock_guard<std::mutex> lk(m->mu);
  auto it = a->live.upper_bound(off);
  if (it == a->live.begin()) return fail(ODC_ERR_NOT_FOUND, "pointer %p is not in a live allocation", ptr);
  --it;
  if (off >= it->first + it->second)
    return fail(ODC_ERR_NOT_FOUND, "pointer %p is not in a live allocation", ptr);
  if (rank) *rank = r;
  if (alloc_offset) *alloc_offset = it->first;
  if (inner) *inner = off - it->first;
  return ODC_OK;
}

// ------------------------------------------------------------------------------------------------
// launches
// ------------------------------------------------------------------------------------------------
}  // extern "C"

namespace {

int dtype_bytes(int dt) {
  switch (dt) {
    case ODC_DTYPE_BF16: return 2;
    case ODC_DTYPE_F16: return 2;
    case ODC_DTYPE_F32: return 4;
    default: return 0;
  }
}

// odc_tiles::fill_tile_table with its failure turned into an error message.
// `order`, when given, maps positions of the launch order to the caller's item indices (for the
// message only: units and take already work on positions).
template <class Units, class Take>
int fill_launch(TileTable& tt, uint32_t world, uint32_t n_items, uint32_t* next, uint64_t tile_units,
                Units units, Take take, const uint32_t* order = nullptr) {
  const int n = fill_tile_table(tt, world, n_items, next, tile_units, units, take);
  if (n < 0) {
    const uint32_t at = (uint32_t)(-1 - n);
    return fail(ODC_ERR_INVALID, "item %u: %llu units per rank is too large for one launch", order ? order[at] : at,
                (unsigned long long)units(at));
  }
  return n;
}

int check_rank_range(const odc_arena* a, const char* what, uint32_t i, uint64_t offset, uint64_t nbytes) {
  if (offset > a->bytes_per_rank || nbytes > a->bytes_per_rank - offset)
    return fail(ODC_ERR_INVALID, "%s %u: [%llu, +%llu) leaves the %llu byte rank region", what, i,
                (unsigned long long)offset, (unsigned long long)nbytes,
                (unsigned long long)a->bytes_per_rank);
  return ODC_OK;
}

// The same for `elems` elements of `elem_bytes` each; an element count whose byte size would wrap
// around is rejected before it is multiplied.
int check_rank_elems(const odc_arena* a, const char* what, uint32_t i, uint64_t offset, uint64_t elems,
                     uint64_t elem_bytes) {
  if (elems > a->bytes_per_rank / elem_bytes)
    return fail(ODC_ERR_INVALID, "%s %u: %llu elements of %llu bytes exceed the %llu byte rank region", what, i,
                (unsigned long long)elems, (unsigned long long)elem_bytes, (unsigned long long)a->bytes_per_rank);
  return check_rank_range(a, what, i, offset, elems * elem_bytes);
}

// dst [d0, d0 + world*seg_bytes) must not overlap any rank's source range at src_offset.
int check_no_overlap(const odc_arena* a, uint32_t i, const void* dst, uint64_t dst_seg_bytes,
                     uint64_t src_offset, uint64_t src_seg_bytes) {
  const uint8_t* d0 = static_cast<const uint8_t*>(dst);
  const uint8_t* d1 = d0 + dst_seg_bytes * a->world;
  if (d1 <= a->origin || d0 >= a->origin + a->rank_stride * a->world) return ODC_OK;
  for (uint32_t r = 0; r < a->world; ++r) {
    const uint8_t* s0 = a->origin + (uint64_t)r * a->rank_stride + src_offset;
    if (d0 < s0 + src_seg_bytes && s0 < d1)
      return fail(ODC_ERR_INVALID, "item %u: dst overlaps rank %u's shard", i, r);
  }
  return ODC_OK;
}

}  // namespace

extern "C" {

int odc_gather(odc_arena* a, const odc_gather_item* items, uint32_t n_items, uint32_t first_rank,
               void* stream) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_items && !items) return fail(ODC_ERR_INVALID, "items is NULL");
  if (first_rank >= a->world)
    return fail(ODC_ERR_INVALID, "first_rank %u >= world size %u", first_rank, a->world);
  for (uint32_t i = 0; i < n_items; ++i) {
    const odc_gather_item& it = items[i];
    if (it.shard_bytes == 0) continue;
    if (!it.dst) return fail(ODC_ERR_INVALID, "item %u: dst is NULL", i);
    if (int rc = check_rank_range(a, "item", i, it.src_offset, it.shard_bytes)) return rc;
    if (int rc = check_no_overlap(a, i, it.dst, it.shard_bytes, it.src_offset, it.shard_bytes)) return rc;
  }
  const Options opt = options_snapshot();
  uint32_t next = 0;
  while (next < n_items) {
    GatherLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    L.tt.order = (uint32_t)opt.rank_major;
    L.tt.first_rank = first_rank;
    const int n = fill_launch(
        L.tt, a->world, n_items, &next, kTileBytes, [&](uint32_t i) { return items[i].shard_bytes; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {static_cast<uint8_t*>(items[i].dst), items[i].src_offset, items[i].shard_bytes};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    bool ragged = false;
    for (uint32_t k = 0; k < L.tt.n_items; ++k)
      ragged |= (((uintptr_t)L.item[k].dst | L.item[k].src_off | L.item[k].seg_bytes) & 15u) != 0;
    const uint32_t grid = grid_for(a, opt.gather_blocks_per_cu, L.tt.n_tiles, ragged);
    const uint32_t lds = lds_claim_for(a, opt.gather_resident_cap, grid, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] { return odc_device::launch_gather(L, grid, lds, stream); })) return rc;
  }
  return ODC_OK;
}

int odc_gather_cast(odc_arena* a, const odc_gather_cast_item* items, uint32_t n_items,
                    int src_dtype, int dst_dtype, uint32_t first_rank, void* stream) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_items && !items) return fail(ODC_ERR_INVALID, "items is NULL");
  if (first_rank >= a->world)
    return fail(ODC_ERR_INVALID, "first_rank %u >= world size %u", first_rank, a->world);
  const int sb = dtype_bytes(src_dtype), db = dtype_bytes(dst_dtype);
  if (!sb || !db) return fail(ODC_ERR_INVALID, "unknown dtype code (src %d, dst %d)", src_dtype, dst_dtype);
  if (!odc_device::has_cast_gather(src_dtype, dst_dtype)) return fail(ODC_ERR_UNSUPPORTED, "gather from dtype %d into dtype %d is not implemented", src_dtype, dst_dtype);
  for (uint32_t i = 0; i < n_items; ++i) {
    const odc_gather_cast_item& it = items[i];
    if (it.shard_elems == 0) continue;
    if (!it.dst) return fail(ODC_ERR_INVALID, "item %u: dst is NULL", i);
    if (it.shard_elems > a->bytes_per_rank / sb)
      return fail(ODC_ERR_INVALID, "item %u: shard of %llu elements exceeds the rank region", i,
                  (unsigned long long)it.shard_elems);
    if (it.src_offset % sb || (uintptr_t)it.dst % db)
      return fail(ODC_ERR_INVALID, "item %u: src_offset or dst is not aligned to its dtype", i);
    if (int rc = check_rank_elems(a, "item", i, it.src_offset, it.shard_elems, sb)) return rc;
    if (int rc = check_no_overlap(a, i, it.dst, it.shard_elems * db, it.src_offset, it.shard_elems * sb)) return rc;
  }
  const Options opt = options_snapshot();
  uint32_t next = 0;
  while (next < n_items) {
    CastGatherLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    L.tt.order = (uint32_t)opt.rank_major;
    L.tt.first_rank = first_rank;
    const int n = fill_launch(
        L.tt, a->world, n_items, &next, kTileElems, [&](uint32_t i) { return items[i].shard_elems; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {static_cast<uint8_t*>(items[i].dst), items[i].shard_elems * (uint64_t)db,
                          items[i].src_offset, items[i].shard_elems};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    const uint32_t grid = grid_for(a, opt.gather_blocks_per_cu, L.tt.n_tiles);
    const uint32_t lds = lds_claim_for(a, opt.cast_resident_cap, grid, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] {
          return odc_device::launch_cast_gather(src_dtype, dst_dtype, L, grid, lds, stream);
        }))
      return rc;
  }
  return ODC_OK;
}

int odc_convert(odc_arena* a, const odc_convert_item* items, uint32_t n_items, int src_dtype,
                int dst_dtype, void* stream) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_items && !items) return fail(ODC_ERR_INVALID, "items is NULL");
  const int sb = dtype_bytes(src_dtype), db = dtype_bytes(dst_dtype);
  if (!sb || !db) return fail(ODC_ERR_INVALID, "unknown dtype code (src %d, dst %d)", src_dtype, dst_dtype);
  if (!odc_device::has_cast_gather(src_dtype, dst_dtype))
    return fail(ODC_ERR_UNSUPPORTED, "conversion from dtype %d into dtype %d is not implemented", src_dtype, dst_dtype);
  for (uint32_t i = 0; i < n_items; ++i) {
    const odc_convert_item& it = items[i];
    if (it.elems == 0) continue;
    if (it.src_offset % sb || it.dst_offset % db)
      return fail(ODC_ERR_INVALID, "item %u: src_offset or dst_offset is not aligned to its dtype", i);
    if (int rc = check_rank_elems(a, "item (source)", i, it.src_offset, it.elems, sb)) return rc;
    if (int rc = check_rank_elems(a, "item (destination)", i, it.dst_offset, it.elems, db)) return rc;
    // the two ranges lie in the same rank region, in every region: they must not touch
    if (it.dst_offset < it.src_offset + it.elems * sb && it.src_offset < it.dst_offset + it.elems * db)
      return fail(ODC_ERR_INVALID, "item %u: the destination overlaps the source", i);
  }
  const Options opt = options_snapshot();
  uint32_t next = 0;
  while (next < n_items) {
    CastGatherLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    L.tt.order = (uint32_t)opt.rank_major;
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, a->world, n_items, &next, kTileElems, [&](uint32_t i) { return items[i].elems; },
        [&](uint32_t slot, uint32_t i) {
          // the gather-with-cast kernel with every rank's output in that rank's own region
          L.item[slot] = {a->origin + items[i].dst_offset, a->rank_stride, items[i].src_offset, items[i].elems};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    const uint32_t grid = grid_for(a, opt.gather_blocks_per_cu, L.tt.n_tiles);
    const uint32_t lds = lds_claim_for(a, opt.cast_resident_cap, grid, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] {
          return odc_device::launch_cast_gather(src_dtype, dst_dtype, L, grid, lds, stream);
        }))
      return rc;
  }
  return ODC_OK;
}

int odc_clear(odc_arena* a, const odc_span* spans, uint32_t n_spans, void* stream) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_spans && !spans) return fail(ODC_ERR_INVALID, "spans is NULL");
  for (uint32_t i = 0; i < n_spans; ++i)
    if (int rc = check_rank_range(a, "span", i, spans[i].offset, spans[i].nbytes)) return rc;
  const Options opt = options_snapshot();
  uint32_t next = 0;
  while (next < n_spans) {
    ClearLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    // a write-only stream runs fastest with the ranks interleaved (measured after an accumulate, as
    // in a step: 117 us at W=64 against 123 item-major and 127 rank-outermost; level at W=128)
    L.tt.order = kRanksInterleaved;
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, a->world, n_spans, &next, kTileBytes, [&](uint32_t i) { return spans[i].nbytes; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {spans[i].offset, spans[i].nbytes};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    const uint32_t grid = grid_for(a, opt.clear_blocks_per_cu, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] { return odc_device::launch_clear(L, grid, stream); })) return rc;
  }
  return ODC_OK;
}

}  // extern "C"
namespace {

// odc_scatter_accumulate (store == false) and odc_scatter_store (store == true)
int scatter_launch(odc_arena* a, const odc_accum_item* items, uint32_t n_items, int grad_dtype,
                   int acc_dtype, void* stream, bool store) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_items && !items) return fail(ODC_ERR_INVALID, "items is NULL");
  const int gb = dtype_bytes(grad_dtype), ab = dtype_bytes(acc_dtype);
  if (!gb || !ab) return fail(ODC_ERR_INVALID, "unknown dtype code (grad %d, acc %d)", grad_dtype, acc_dtype);
  if (!odc_device::has_accum(grad_dtype, acc_dtype))
    return fail(ODC_ERR_UNSUPPORTED, "scatter-accumulate of grad dtype %d into acc dtype %d is not implemented",
                grad_dtype, acc_dtype);
  for (uint32_t i = 0; i < n_items; ++i) {
    const odc_accum_item& it = items[i];
    if (it.shard_elems == 0) {
      if (it.grad_elems) return fail(ODC_ERR_INVALID, "item %u: grad_elems > 0 with shard_elems == 0", i);
      continue;
    }
    if (it.shard_elems > a->bytes_per_rank / ab)
      return fail(ODC_ERR_INVALID, "item %u: shard of %llu elements exceeds the rank region", i,
                  (unsigned long long)it.shard_elems);
    if (it.acc_offset % ab)
      return fail(ODC_ERR_INVALID, "item %u: acc_offset %llu is not aligned to the accumulation dtype", i,
                  (unsigned long long)it.acc_offset);
    if (int rc = check_rank_elems(a, "item", i, it.acc_offset, it.shard_elems, ab)) return rc;
    if (it.grad_elems > it.shard_elems * a->world)
      return fail(ODC_ERR_INVALID, "item %u: grad_elems %llu > world_size * shard_elems = %llu", i,
                  (unsigned long long)it.grad_elems, (unsigned long long)(it.shard_elems * a->world));
    if (it.grad_elems && !it.grad) return fail(ODC_ERR_INVALID, "item %u: grad is NULL", i);
    if ((uintptr_t)it.grad % gb)
      return fail(ODC_ERR_INVALID, "item %u: grad pointer is not aligned to the gradient dtype", i);
  }
  const Options opt = options_snapshot();
  // Launch order of the items: those of less than one tile per rank go last. A tiny segment
  // between two long ones (a norm vector's 64-element slice between two projection matrices)
  // slows the read-modify-write stream around it out of all proportion to its size; at the end
  // of the list it costs nothing (measured on the 8B layer, 9 items: -0.6 % of the launch time at
  // W=64, -1.2 % at W=32, -5 % at W=128, nothing at W=8, where there are 16 such tiles instead of
  // 128 or more; the gathers, the clear and the store form do not care). Items of one call are
  // disjoint, so their order never changes the result.
  uint32_t order_inline[256];
  std::vector<uint32_t> order_heap;
  uint32_t* order = order_inline;
  if (n_items > 256) {
    order_heap.resize(n_items);
    order = order_heap.data();
  }
  {
    uint32_t k = 0;
    for (int small = 0; small < 2; ++small)
      for (uint32_t i = 0; i < n_items; ++i)
        if ((opt.accum_small_items_last != 0 && items[i].shard_elems < kTileElems) == (small != 0)) order[k++] = i;
  }
  uint32_t next = 0;
  while (next < n_items) {
    AccumLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    L.tt.order = (uint32_t)opt.rank_major;
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, a->world, n_items, &next, kTileElems, [&](uint32_t i) { return items[order[i]].shard_elems; },
        [&](uint32_t slot, uint32_t i) {
          const odc_accum_item& it = items[order[i]];
          L.item[slot] = {static_cast<const uint8_t*>(it.grad), it.grad_elems, it.acc_offset, it.shard_elems};
        },
        order);
    if (n < 0) return n;
    if (n == 0) continue;
    // Tile order. Item-major (a rank's segment, then the next rank's, item by item) walks the
    // gradient contiguously and hops between rank regions at every segment; rank-outermost walks
    // one rank region from accumulation to accumulation (they are neighbours when registered
    // together) and hops in the gradient instead. The read-modify-write stream is the one worth
    // keeping contiguous once segments get short. Measured on the 8B layer, item-major against
    // rank-outermost: +1.1 % at W=4, +1.6 % at W=16 (370 tiles per segment on average), -1.9 % at
    // W=32 (185), -6 % at W=64, -10 % at W=128.
    const uint64_t segments = (uint64_t)L.tt.n_items * a->world;
    if (opt.accum_tile_order == 3)
      L.tt.order = L.tt.n_tiles < (uint64_t)opt.accum_short_segment_tiles * segments ? kRankOutermost : kItemMajor;
    else
      L.tt.order = (uint32_t)opt.accum_tile_order;
    // Launch shape: one workgroup per tile. A persistent shape (one workgroup per CU,
    // "accum_blocks_per_cu" = 1, or automatically below "accum_persistent_below_tiles" tiles per
    // segment) used to win on very short segments (+1.6 % at W=64) only because it suffered less
    // from tiny segments in the middle of the tile order; with those moved to the end the two
    // shapes are level at W=64 and W=128 and one workgroup per tile is ahead everywhere else
    // (W=16: +1.5 %, W=32: +0.9 %), and it is the shape that co-runs with compute kernels
    // without starving them. A persistent grid is never used for ragged launches (a lone
    // workgroup that straddles lines or meets heads, tails and padding falls behind: -7 % on
    // 16 B aligned uneven shards) nor for other dtype pairs than 16-bit gradients into fp32.
    bool ragged = !(gb == 2 && ab == 4);
    for (uint32_t k = 0; k < L.tt.n_items; ++k)
      ragged |= (L.item[k].acc_off & 127u) != 0 || ((L.item[k].seg_elems * ab) & 127u) != 0 ||
                ((L.item[k].seg_elems * gb) & 127u) != 0 || ((uintptr_t)L.item[k].grad & 127u) != 0 ||
                L.item[k].grad_elems != L.item[k].seg_elems * a->world;
    int64_t blocks_per_cu = store ? opt.store_blocks_per_cu : opt.accum_blocks_per_cu;
    if (blocks_per_cu < 0)
      blocks_per_cu = L.tt.n_tiles < (uint64_t)opt.accum_persistent_below_tiles * segments ? 1 : 0;
    const uint32_t grid = grid_for(a, blocks_per_cu, L.tt.n_tiles, ragged);
    const int64_t cap = store ? opt.store_resident_cap : opt.accum_resident_cap;
    const uint32_t lds = lds_claim_for(a, cap, grid, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] {
          return odc_device::launch_accum(grad_dtype, acc_dtype, store, L, grid, lds, stream);
        }))
      return rc;
  }
  return ODC_OK;
}

}  // namespace

extern "C" {

int odc_scatter_accumulate(odc_arena* a, const odc_accum_item* items, uint32_t n_items,
                           int grad_dtype, int acc_dtype, void* stream) {
  return scatter_launch(a, items, n_items, grad_dtype, acc_dtype, stream, false);
}

int odc_scatter_store(odc_arena* a, const odc_accum_item* items, uint32_t n_items, int grad_dtype,
                      int acc_dtype, void* stream) {
  return scatter_launch(a, items, n_items, grad_dtype, acc_dtype, stream, true);
}

int odc_publish(odc_arena* a, uint32_t rank, const odc_publish_item* items, uint32_t n_items,
                int acc_dtype, int out_dtype, float divisor, void* stream) {
  DeviceGuard guard;
  if (int rc = check_compute(a, guard)) return rc;
  if (n_items && !items) return fail(ODC_ERR_INVALID, "items is NULL");
  if (rank >= a->world) return fail(ODC_ERR_INVALID, "rank %u >= world size %u", rank, a->world);
  const int ab = dtype_bytes(acc_dtype), ob = dtype_bytes(out_dtype);
  if (!ab || !ob) return fail(ODC_ERR_INVALID, "unknown dtype code (acc %d, out %d)", acc_dtype, out_dtype);
  if (!(divisor == divisor) || divisor == 0.0f) return fail(ODC_ERR_INVALID, "divisor must be a non-zero number");
  if (!odc_device::has_publish(acc_dtype, out_dtype)) return fail(ODC_ERR_UNSUPPORTED, "publish from dtype %d into dtype %d is not implemented", acc_dtype, out_dtype);
  uint8_t* region = a->origin + (uint64_t)rank * a->rank_stride;
  for (uint32_t i = 0; i < n_items; ++i) {
    const odc_publish_item& it = items[i];
    if (it.elems == 0) continue;
    if (it.elems > a->bytes_per_rank / ab)
      return fail(ODC_ERR_INVALID, "item %u: %llu elements exceed the rank region", i, (unsigned long long)it.elems);
    if (it.acc_offset % ab || (uintptr_t)it.out % ob)
      return fail(ODC_ERR_INVALID, "item %u: acc_offset or out is not aligned to its dtype", i);
    if (int rc = check_rank_range(a, "item", i, it.acc_offset, it.elems * ab)) return rc;
    if (it.out) {
      const uint8_t* o0 = static_cast<const uint8_t*>(it.out);
      const uint8_t* s0 = region + it.acc_offset;
      if (o0 < s0 + it.elems * ab && s0 < o0 + it.elems * ob)
        return fail(ODC_ERR_INVALID, "item %u: out overlaps the accumulation it is published from", i);
    }
  }
  const Options opt = options_snapshot();
  uint32_t next = 0;
  while (next < n_items) {
    PublishLaunch L;
    L.region = region;
    L.divisor = divisor;
    L.divide = divisor != 1.0f;
    L.reciprocal = 1.0f;
    // Dividing by a power of two whose reciprocal is a normal number is the same correctly
    // rounded result as multiplying by that reciprocal (both round one exact real value), and
    // costs one instruction instead of the division sequence.
    int exponent = 0;
    if (L.divide && std::fabs(std::frexp(divisor, &exponent)) == 0.5f && exponent > -120 && exponent < 120) {
      L.reciprocal = 1.0f / divisor;
      L.divide = 2;
    }
    L.tt.order = kItemMajor;
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, 1u, n_items, &next, kTileElems, [&](uint32_t i) { return items[i].elems; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {static_cast<uint8_t*>(items[i].out), items[i].acc_offset, items[i].elems};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    // one workgroup per tile: the division sequence wants the occupancy, and the launch is short
    const uint32_t grid = grid_for(a, opt.publish_blocks_per_cu, L.tt.n_tiles);
    const uint32_t lds = lds_claim_for(a, opt.publish_resident_cap, grid, L.tt.n_tiles);
    if (int rc = launch_tiles(a, L, grid, [&] {
          return odc_device::launch_publish(acc_dtype, out_dtype, L, grid, lds, stream);
        }))
      return rc;
  }
  return ODC_OK;
}

}  // extern "C"
