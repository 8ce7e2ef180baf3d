// libodc_hip.so — gfx950 (MI355X, CDNA4) implementation of the C ABI in include/odc_hip.h.
//
// Five streaming kernels, all HBM-bandwidth bound (no MFMA, no LDS):
//   gather_kernel       : W shard regions -> one flat buffer          (read 1 B + write 1 B per byte)
//   cast_gather_kernel  : the same with a dtype conversion on the way (fp32 -> bf16: 6 B per element)
//   accum_kernel        : acc_r += widen(grad chunk r), in place      (bf16 -> fp32: 10 B per element)
//                         or acc_r = +0 + widen(grad chunk r), acc not read          (6 B per element)
//   clear_kernel        : zero a span in every rank region            (write 1 B per byte)
//   publish_kernel      : one rank's acc /= divisor, plus a cast copy (end of a minibatch)
// plus the host-side symmetric arena (one hipMalloc, W rank regions, one offset valid in all).
//
// Launch model shared by the kernels: the work of one launch is cut into tiles of
// kThreads * kUnroll = 1024 vectors (16 KiB); workgroups of 256 threads (512 for the two
// gathers and the scatter-store) walk the tiles with a grid-stride loop, by default one workgroup per tile, so that,
// at any instant, the whole chip streams one compact window of memory. Per-item
// descriptors (<= ODC_MAX_ITEMS_PER_LAUNCH) travel BY VALUE in the kernel argument segment and
// are read with scalar loads, so a call needs no device-side work list, no host->device copy and
// no allocation; longer item lists are split over several launches.
//
// Each wavefront issues its 2 or 4 independent 128-bit nontemporal loads per stream before the
// first store: on this part the nontemporal hint on both loads and stores is worth ~15 % over
// plain accesses for these single-touch streams. Deeper unrolling or prefetching the next tile
// measured slower: the memory system prefers a small window to more requests in flight.
// Workgroup i runs on XCD i % 8; binding XCDs to address classes (256 B .. 64 KiB granules)
// changed nothing measurable and giving every XCD one contiguous eighth of the tiles costs the
// read-modify-write 3 %, so tiles are simply dealt out in address order: at any instant all
// eight XCDs work side by side in one window of memory.

#include <hip/hip_runtime.h>

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

#include "odc_hip.h"
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

#define ODC_HIP_TRY(expr)                                                                   \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    if (e_ != hipSuccess)                                                                   \
      return fail(ODC_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),       \
                  __FILE__, __LINE__);                                                      \
  } while (0)

// ------------------------------------------------------------------------------------------------
// options
// ------------------------------------------------------------------------------------------------
// Workgroup shape of the two gathers and of the scatter-store (the kernels that read one stream
// and write one): 512 threads x 2 steps over the same 16 KiB tile as the 256 x 4 of the other
// kernels. Four such workgroups fill a CU's wave slots, which is the residency these kernels
// stream best at (measured: gathers +1.4..2.6 % over 256 x 4 with a residency cap of 4, which
// had to be enforced by claiming LDS; scatter-store level with it on per-parameter shards at W=8
// and +2..3 % on flat shards and at W=64; 256 x 4 without a cap loses 6..8 %; 1024 x 1 loses
// 20 %). The read-modify-write keeps 256 x 4 (512 x 2: equal on long segments, -3 % in the
// persistent shape at W=64), and so does the clear (512 x 2: -25 % on per-parameter spans).
constexpr int kCopyThreads = 512;
constexpr int kCopyUnroll = (int)odc_tiles::kTileVecs / kCopyThreads;  // 2 for the 16 KiB tile
constexpr int kStoreThreads = 512;
constexpr int kStoreUnroll = (int)odc_tiles::kTileVecs / kStoreThreads;
static_assert(kCopyUnroll >= 1 && kStoreUnroll >= 1, "a tile holds at least one vector per thread");

struct Options {
  // measured on MI355X over a Llama-3-8B layer: every kernel peaks with one workgroup per tile
  // and no residency cap
  int64_t gather_blocks_per_cu = 0;
  int64_t gather_resident_cap = 0;  // 512-thread workgroups: 4 per CU without a cap
  int64_t cast_resident_cap = 0;
  int64_t accum_resident_cap = 0;
  int64_t accum_blocks_per_cu = -1;  // -1: by segment length (see scatter_launch)
  int64_t accum_short_segment_tiles = 256;   // segments averaging fewer tiles: rank-outermost tile order
  int64_t accum_persistent_below_tiles = 128;  // segments averaging fewer tiles: persistent launch shape
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

// ------------------------------------------------------------------------------------------------
// device side
// ------------------------------------------------------------------------------------------------
using namespace odc_tiles;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Per-launch descriptors, passed by value (kernel argument segment, scalar loads): the launch's
// TileTable (odc_tiles.h) and one small record per item.
struct GatherDesc {
  uint8_t* dst;
  uint64_t src_off;
  uint64_t seg_bytes;
};
struct GatherLaunch {
  TileTable tt;
  const uint8_t* base;  // arena base (rank 0 region)
  uint64_t rank_stride;
  GatherDesc item[kMaxItems];
};

struct CastGatherDesc {
  uint8_t* dst;
  uint64_t src_off;
  uint64_t seg_elems;
};
struct CastGatherLaunch {
  TileTable tt;
  const uint8_t* base;
  uint64_t rank_stride;
  CastGatherDesc item[kMaxItems];
};

struct AccumDesc {
  const uint8_t* grad;
  uint64_t grad_elems;
  uint64_t acc_off;
  uint64_t seg_elems;
};
struct AccumLaunch {
  TileTable tt;
  uint8_t* base;
  uint64_t rank_stride;
  AccumDesc item[kMaxItems];
};

struct ClearDesc {
  uint64_t off;
  uint64_t seg_bytes;
};
struct ClearLaunch {
  TileTable tt;
  uint8_t* base;
  uint64_t rank_stride;
  ClearDesc item[kMaxItems];
};

struct PublishDesc {
  uint8_t* out;  // may be null: divide in place only
  uint64_t acc_off;
  uint64_t seg_elems;
};
struct PublishLaunch {  // one rank's region only: tt.world == 1
  TileTable tt;
  uint8_t* region;      // base of the publishing rank's region
  float divisor;
  float reciprocal;     // exact 1 / divisor when divide == 2
  uint32_t divide;      // 0: leave the accumulation untouched, 1: divide, 2: multiply by reciprocal
  PublishDesc item[kMaxItems];
};
static_assert(sizeof(GatherLaunch) <= 4096 && sizeof(AccumLaunch) <= 4096 && sizeof(PublishLaunch) <= 4096 &&
                  sizeof(CastGatherLaunch) <= 4096 && sizeof(ClearLaunch) <= 4096,
              "launch descriptors must fit the kernel-argument segment");

// The read side of a tile takes whatever misalignment the written side's alignment leaves it
// with; these typedefs tell the compiler so.
typedef u32x4 u32x4_u __attribute__((aligned(1)));
typedef u32x2 u32x2_u __attribute__((aligned(1)));

template <class V> struct Unaligned;
template <> struct Unaligned<u32x4> { typedef u32x4_u type; };
template <> struct Unaligned<u32x2> { typedef u32x2_u type; };

template <class V>
__device__ __forceinline__ V load_stream(const uint8_t* p) {  // nontemporal, any alignment
  return __builtin_nontemporal_load(reinterpret_cast<const typename Unaligned<V>::type*>(p));
}

// ---- gather -------------------------------------------------------------------------------
// Everything of a tile that is not a run of kTileVecs whole vectors: the last partial run, the
// head and the tail. Kept out of line so that the streaming loop stays tight.
template <int T, int U>
__device__ __attribute__((noinline)) void gather_edges(uint8_t* d, const uint8_t* s, uint32_t chunk, SegShape g) {
  // Every load of the tile is issued before its first store (a lone resident workgroup would
  // otherwise pay one memory round trip per step).
  const uint32_t tid = threadIdx.x;
  const TileWork w = tile_work(chunk, g);
  const uint32_t left = is_whole(w) ? 0u : w.nv;
  const uint8_t* sb = s + g.head + w.v0 * 16;
  u32x4* db = reinterpret_cast<u32x4*>(d + g.head) + w.v0;
  const bool do_head = w.head && tid < g.head;
  const bool do_tail = w.tail && tid < g.tail;
  const uint64_t tail_at = g.head + g.nvec * 16 + tid;
  u32x4 v[U];
  uint8_t head_byte = 0, tail_byte = 0;
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (u * T + tid < left) v[u] = load_stream<u32x4>(sb + (size_t)(u * T + tid) * 16);
  if (do_head) head_byte = s[tid];
  if (do_tail) tail_byte = s[tail_at];
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (u * T + tid < left) __builtin_nontemporal_store(v[u], db + u * T + tid);
  if (do_head) d[tid] = head_byte;
  if (do_tail) d[tail_at] = tail_byte;
}

// T threads do a tile in U steps of T vectors (T * U = kTileVecs, so the geometry is that of every
// other kernel); the copies stream best from 512-thread workgroups, of which 4 fit a CU.
template <int T, int U>
__global__ __launch_bounds__(T) void gather_kernel(const GatherLaunch launch) {
  static_assert(T * U == (int)kTileVecs, "one tile per workgroup step");
  const uint32_t tid = threadIdx.x;
  TileCursor cur;
  GatherDesc it = {};
  for (uint32_t t = blockIdx.x; t < launch.tt.n_tiles; t += gridDim.x) {
    if (!cursor_holds(cur, t)) {
      cursor_seek(launch.tt, t, cur);
      it = launch.item[cur.item];  // issued together with the loads of cursor_enter
      cursor_enter(launch.tt, cur);
    }
    const TileCoord c = cursor_coord(launch.tt, cur, t);
    const uint64_t seg = it.seg_bytes;
    const uint8_t* s = launch.base + (uint64_t)c.rank * launch.rank_stride + it.src_off;
    uint8_t* d = it.dst + (uint64_t)c.rank * seg;
    const SegShape g = seg_shape((uintptr_t)d, seg, 1, 16);
    const TileWork w = tile_work(c.chunk, g);
    if (is_whole(w)) {
      const uint8_t* sb = s + g.head + (w.v0 + tid) * 16;
      u32x4* db = reinterpret_cast<u32x4*>(d + g.head) + w.v0 + tid;
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = load_stream<u32x4>(sb + (size_t)u * T * 16);
      // a whole tile that also owns its segment's head or tail (the first and last tile of a
      // ragged segment) reads those bytes with the same round trip as its vectors
      const bool do_head = w.head && tid < g.head;
      const bool do_tail = w.tail && tid < g.tail;
      const uint64_t tail_at = g.head + g.nvec * 16 + tid;
      uint8_t head_byte = 0, tail_byte = 0;
      if (do_head) head_byte = s[tid];
      if (do_tail) tail_byte = s[tail_at];
#pragma unroll
      for (int u = 0; u < U; ++u) __builtin_nontemporal_store(v[u], db + u * T);
      if (do_head) d[tid] = head_byte;
      if (do_tail) d[tail_at] = tail_byte;
    } else if (has_edges(w)) {
      gather_edges<T, U>(d, s, c.chunk, g);
    }
  }
}

// ---- clear --------------------------------------------------------------------------------
// Plain (not nontemporal) stores: for a write-only stream they measure faster here.
__device__ __attribute__((noinline)) void clear_edges(uint8_t* d, uint32_t chunk, SegShape g) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const uint32_t tid = threadIdx.x;
  const TileWork w = tile_work(chunk, g);
  if (!is_whole(w)) {
    u32x4* db = reinterpret_cast<u32x4*>(d + g.head) + w.v0;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (u * kThreads + tid < w.nv) db[u * kThreads + tid] = zero;
  }
  if (w.head && tid < g.head) d[tid] = 0;
  if (w.tail && tid < g.tail) d[g.head + g.nvec * 16 + tid] = 0;
}

__global__ __launch_bounds__(kThreads) void clear_kernel(const ClearLaunch launch) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
  const uint32_t tid = threadIdx.x;
  TileCursor cur;
  ClearDesc it = {};
  for (uint32_t t = blockIdx.x; t < launch.tt.n_tiles; t += gridDim.x) {
    if (!cursor_holds(cur, t)) {
      cursor_seek(launch.tt, t, cur);
      it = launch.item[cur.item];  // issued together with the loads of cursor_enter
      cursor_enter(launch.tt, cur);
    }
    const TileCoord c = cursor_coord(launch.tt, cur, t);
    uint8_t* d = launch.base + (uint64_t)c.rank * launch.rank_stride + it.off;
    const SegShape g = seg_shape((uintptr_t)d, it.seg_bytes, 1, 16);
    const TileWork w = tile_work(c.chunk, g);
    if (is_whole(w)) {
      u32x4* db = reinterpret_cast<u32x4*>(d + g.head) + w.v0 + tid;
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) db[u * kThreads] = zero;
    }
    if (has_edges(w)) clear_edges(d, c.chunk, g);
  }
}

// ---- scatter-accumulate -------------------------------------------------------------------
// Element codecs. Widening to fp32 is exact for all three types; narrowing rounds to nearest
// even. The add itself is one v_add_f32 per element: no contraction, no reassociation.
struct bf16_tag {};
struct f16_tag {};
struct f32_tag {};

template <class T> struct Codec;
template <> struct Codec<f32_tag> {
  static constexpr int kBytes = 4;
  typedef uint32_t raw_t;
  static __device__ __forceinline__ float widen(uint32_t r) { return __uint_as_float(r); }
  static __device__ __forceinline__ uint32_t narrow(float f) { return __float_as_uint(f); }
};
template <> struct Codec<bf16_tag> {
  static constexpr int kBytes = 2;
  typedef uint16_t raw_t;
  static __device__ __forceinline__ float widen(uint16_t r) { return __uint_as_float((uint32_t)r << 16); }
  static __device__ __forceinline__ uint16_t narrow(float f) {
    const uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;  // NaN
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
};
template <> struct Codec<f16_tag> {
  static constexpr int kBytes = 2;
  typedef uint16_t raw_t;
  static __device__ __forceinline__ float widen(uint16_t r) {
    return (float)__builtin_bit_cast(_Float16, r);
  }
  static __device__ __forceinline__ uint16_t narrow(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
};

// Four consecutive elements as raw dwords: 2 dwords for the 16-bit types, 4 for fp32.
template <class T> struct Quad;
template <> struct Quad<f32_tag> {
  typedef u32x4 vec_t;
  static __device__ __forceinline__ void widen(vec_t r, float (&f)[4]) {
    f[0] = __uint_as_float(r.x); f[1] = __uint_as_float(r.y);
    f[2] = __uint_as_float(r.z); f[3] = __uint_as_float(r.w);
  }
  static __device__ __forceinline__ vec_t narrow(const float (&f)[4]) {
    vec_t r = {__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    return r;
  }
};
template <> struct Quad<bf16_tag> {
  typedef u32x2 vec_t;
  static __device__ __forceinline__ void widen(vec_t r, float (&f)[4]) {
    f[0] = __uint_as_float(r.x << 16); f[1] = __uint_as_float(r.x & 0xffff0000u);
    f[2] = __uint_as_float(r.y << 16); f[3] = __uint_as_float(r.y & 0xffff0000u);
  }
  static __device__ __forceinline__ vec_t narrow(const float (&f)[4]) {
    vec_t r;
    r.x = (uint32_t)Codec<bf16_tag>::narrow(f[0]) | ((uint32_t)Codec<bf16_tag>::narrow(f[1]) << 16);
    r.y = (uint32_t)Codec<bf16_tag>::narrow(f[2]) | ((uint32_t)Codec<bf16_tag>::narrow(f[3]) << 16);
    return r;
  }
};
template <> struct Quad<f16_tag> {
  typedef u32x2 vec_t;
  static __device__ __forceinline__ void widen(vec_t r, float (&f)[4]) {
    f[0] = Codec<f16_tag>::widen((uint16_t)(r.x & 0xffffu)); f[1] = Codec<f16_tag>::widen((uint16_t)(r.x >> 16));
    f[2] = Codec<f16_tag>::widen((uint16_t)(r.y & 0xffffu)); f[3] = Codec<f16_tag>::widen((uint16_t)(r.y >> 16));
  }
  static __device__ __forceinline__ vec_t narrow(const float (&f)[4]) {
    vec_t r;
    r.x = (uint32_t)Codec<f16_tag>::narrow(f[0]) | ((uint32_t)Codec<f16_tag>::narrow(f[1]) << 16);
    r.y = (uint32_t)Codec<f16_tag>::narrow(f[2]) | ((uint32_t)Codec<f16_tag>::narrow(f[3]) << 16);
    return r;
  }
};

// kStore: the accumulation is taken to hold +0 and is not read (acc = +0 + g, the value a clear
// followed by an accumulate leaves: -0 gradients still become +0).
//
// The parts of a tile that are not whole runs of valid quads: a partial last run, a run that
// crosses the end of the valid gradient or lies in the zero padding, the head and the tail.
// Gradient elements at index >= grad_elems read as +0 and are still added (so an accumulation
// holding -0 becomes +0, as F.pad followed by add_ leaves it). Two phases, every load of the tile
// before its first store: a lone resident workgroup would otherwise pay one memory round trip
// per quad.
template <class G, class A, bool kStore, int T, int U>
__device__ __attribute__((noinline)) void accum_edges(uint8_t* acc, const uint8_t* grad, uint64_t g_seg,
                                                      uint64_t grad_elems, uint32_t chunk, SegShape g,
                                                      bool body) {
  typedef typename Quad<G>::vec_t gvec_t;
  typedef typename Quad<A>::vec_t avec_t;
  typedef typename Codec<G>::raw_t graw_t;
  typedef typename Codec<A>::raw_t araw_t;
  constexpr uint32_t kAB = Codec<A>::kBytes, kGB = Codec<G>::kBytes;
  const uint32_t tid = threadIdx.x;
  const TileWork w = tile_work(chunk, g);
  const uint32_t left = body ? w.nv : 0u;
  const uint64_t e0 = g.head + w.v0 * 4;
  avec_t* ap = reinterpret_cast<avec_t*>(acc + e0 * kAB);
  const graw_t* gs = reinterpret_cast<const graw_t*>(grad);
  araw_t* as = reinterpret_cast<araw_t*>(acc);
  const bool do_head = w.head && tid < g.head;
  const bool do_tail = w.tail && tid < g.tail;
  const uint64_t tail_at = g.head + g.nvec * 4 + tid;

  float gf[U][4];
  avec_t araw[U];
  float head_g = 0.0f, head_a = 0.0f, tail_g = 0.0f, tail_a = 0.0f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t q = u * T + tid;
#pragma unroll
    for (int k = 0; k < 4; ++k) gf[u][k] = 0.0f;
    if (q < left) {
      const uint64_t gi = g_seg + e0 + (uint64_t)q * 4;
      if (gi + 4 <= grad_elems) {
        Quad<G>::widen(load_stream<gvec_t>(grad + gi * kGB), gf[u]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (gi + k < grad_elems) gf[u][k] = Codec<G>::widen(gs[gi + k]);
      }
      if constexpr (!kStore) araw[u] = __builtin_nontemporal_load(ap + q);
    }
  }
  if (do_head) {
    if (g_seg + tid < grad_elems) head_g = Codec<G>::widen(gs[g_seg + tid]);
    if constexpr (!kStore) head_a = Codec<A>::widen(as[tid]);
  }
  if (do_tail) {
    if (g_seg + tail_at < grad_elems) tail_g = Codec<G>::widen(gs[g_seg + tail_at]);
    if constexpr (!kStore) tail_a = Codec<A>::widen(as[tail_at]);
  }

#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t q = u * T + tid;
    if (q < left) {
      float af[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (!kStore) Quad<A>::widen(araw[u], af);
#pragma unroll
      for (int k = 0; k < 4; ++k) af[k] = af[k] + gf[u][k];
      __builtin_nontemporal_store(Quad<A>::narrow(af), ap + q);
    }
  }
  if (do_head) as[tid] = Codec<A>::narrow(head_a + head_g);
  if (do_tail) as[tail_at] = Codec<A>::narrow(tail_a + tail_g);
}

template <class G, class A, bool kStore, int T, int U>
__global__ __launch_bounds__(T) void accum_kernel(const AccumLaunch launch) {
  static_assert(T * U == (int)kTileVecs, "one tile per workgroup step");
  typedef typename Quad<G>::vec_t gvec_t;
  typedef typename Quad<A>::vec_t avec_t;
  constexpr uint32_t kAB = Codec<A>::kBytes, kGB = Codec<G>::kBytes;
  const uint32_t tid = threadIdx.x;
  TileCursor cur;
  AccumDesc it = {};
  for (uint32_t t = blockIdx.x; t < launch.tt.n_tiles; t += gridDim.x) {
    if (!cursor_holds(cur, t)) {
      cursor_seek(launch.tt, t, cur);
      it = launch.item[cur.item];  // issued together with the loads of cursor_enter
      cursor_enter(launch.tt, cur);
    }
    const TileCoord c = cursor_coord(launch.tt, cur, t);
    const uint64_t seg = it.seg_elems;
    uint8_t* acc = launch.base + (uint64_t)c.rank * launch.rank_stride + it.acc_off;
    const uint64_t g_seg = (uint64_t)c.rank * seg;  // gradient index of the segment's first element
    const SegShape g = seg_shape((uintptr_t)acc, seg, kAB, 4);
    const TileWork w = tile_work(c.chunk, g);
    const uint64_t e0 = g.head + w.v0 * 4;  // the tile's first body element within the segment
    // whole: all kTileVecs quads exist in the accumulation AND in the valid part of the gradient
    const bool whole = is_whole(w) && g_seg + e0 + kTileElems <= it.grad_elems;
    if (whole) {
      const uint8_t* gb = it.grad + (g_seg + e0) * kGB + (size_t)tid * sizeof(gvec_t);
      avec_t* ap = reinterpret_cast<avec_t*>(acc + e0 * kAB) + tid;
      gvec_t graw[U];
      avec_t araw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) graw[u] = load_stream<gvec_t>(gb + (size_t)u * T * sizeof(gvec_t));
      if constexpr (!kStore) {
#pragma unroll
        for (int u = 0; u < U; ++u) araw[u] = __builtin_nontemporal_load(ap + u * T);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float gf[4], af[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        Quad<G>::widen(graw[u], gf);
        if constexpr (!kStore) Quad<A>::widen(araw[u], af);
#pragma unroll
        for (int k = 0; k < 4; ++k) af[k] = af[k] + gf[k];
        __builtin_nontemporal_store(Quad<A>::narrow(af), ap + u * T);
      }
    }
    if (!whole ? (w.nv != 0 || w.head || w.tail) : (w.head || w.tail))
      accum_edges<G, A, kStore, T, U>(acc, it.grad, g_seg, it.grad_elems, c.chunk, g, !whole);
  }
}

// ---- gather with cast ---------------------------------------------------------------------
// dst[r*S + i] = narrow_D(widen_S(region_r[off + i])): the gather of shards kept in one dtype
// (fp32 master copies) into a full parameter of another (bf16), in one pass.
template <class S, class D, int T, int U>
__device__ __attribute__((noinline)) void cast_edges(uint8_t* d, const uint8_t* s, uint32_t chunk, SegShape g) {
  typedef typename Quad<S>::vec_t svec_t;
  typedef typename Quad<D>::vec_t dvec_t;
  typedef typename Codec<S>::raw_t sraw_t;
  typedef typename Codec<D>::raw_t draw_t;
  constexpr uint32_t kSB = Codec<S>::kBytes, kDB = Codec<D>::kBytes;
  const uint32_t tid = threadIdx.x;
  const TileWork w = tile_work(chunk, g);
  const uint32_t left = is_whole(w) ? 0u : w.nv;
  const uint64_t e0 = g.head + w.v0 * 4;
  const uint8_t* sb = s + e0 * kSB;
  dvec_t* dp = reinterpret_cast<dvec_t*>(d + e0 * kDB);
  const sraw_t* ss = reinterpret_cast<const sraw_t*>(s);
  draw_t* ds = reinterpret_cast<draw_t*>(d);
  const bool do_head = w.head && tid < g.head;
  const bool do_tail = w.tail && tid < g.tail;
  const uint64_t tail_at = g.head + g.nvec * 4 + tid;
  // every load of the tile before its first store
  svec_t raw[U];
  sraw_t head_raw = 0, tail_raw = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t q = u * T + tid;
    if (q < left) raw[u] = load_stream<svec_t>(sb + (size_t)q * sizeof(svec_t));
  }
  if (do_head) head_raw = ss[tid];
  if (do_tail) tail_raw = ss[tail_at];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t q = u * T + tid;
    if (q < left) {
      float f[4];
      Quad<S>::widen(raw[u], f);
      __builtin_nontemporal_store(Quad<D>::narrow(f), dp + q);
    }
  }
  if (do_head) ds[tid] = Codec<D>::narrow(Codec<S>::widen(head_raw));
  if (do_tail) ds[tail_at] = Codec<D>::narrow(Codec<S>::widen(tail_raw));
}

template <class S, class D, int T, int U>
__global__ __launch_bounds__(T) void cast_gather_kernel(const CastGatherLaunch launch) {
  static_assert(T * U == (int)kTileVecs, "one tile per workgroup step");
  typedef typename Quad<S>::vec_t svec_t;
  typedef typename Quad<D>::vec_t dvec_t;
  constexpr uint32_t kSB = Codec<S>::kBytes, kDB = Codec<D>::kBytes;
  const uint32_t tid = threadIdx.x;
  TileCursor cur;
  CastGatherDesc it = {};
  for (uint32_t t = blockIdx.x; t < launch.tt.n_tiles; t += gridDim.x) {
    if (!cursor_holds(cur, t)) {
      cursor_seek(launch.tt, t, cur);
      it = launch.item[cur.item];  // issued together with the loads of cursor_enter
      cursor_enter(launch.tt, cur);
    }
    const TileCoord c = cursor_coord(launch.tt, cur, t);
    const uint64_t seg = it.seg_elems;
    const uint8_t* s = launch.base + (uint64_t)c.rank * launch.rank_stride + it.src_off;
    uint8_t* d = it.dst + (uint64_t)c.rank * seg * kDB;
    const SegShape g = seg_shape((uintptr_t)d, seg, kDB, 4);
    const TileWork w = tile_work(c.chunk, g);
    if (is_whole(w)) {
      const uint64_t e0 = g.head + w.v0 * 4;
      const uint8_t* sb = s + e0 * kSB + (size_t)tid * sizeof(svec_t);
      dvec_t* dp = reinterpret_cast<dvec_t*>(d + e0 * kDB) + tid;
      svec_t raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u) raw[u] = load_stream<svec_t>(sb + (size_t)u * T * sizeof(svec_t));
      // the head and the tail of the segment, when this whole tile owns them, in the same round trip
      typedef typename Codec<S>::raw_t sraw_t;
      typedef typename Codec<D>::raw_t draw_t;
      const sraw_t* ss = reinterpret_cast<const sraw_t*>(s);
      draw_t* ds = reinterpret_cast<draw_t*>(d);
      const bool do_head = w.head && tid < g.head;
      const bool do_tail = w.tail && tid < g.tail;
      const uint64_t tail_at = g.head + g.nvec * 4 + tid;
      sraw_t head_raw = 0, tail_raw = 0;
      if (do_head) head_raw = ss[tid];
      if (do_tail) tail_raw = ss[tail_at];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float f[4];
        Quad<S>::widen(raw[u], f);
        __builtin_nontemporal_store(Quad<D>::narrow(f), dp + u * T);
      }
      if (do_head) ds[tid] = Codec<D>::narrow(Codec<S>::widen(head_raw));
      if (do_tail) ds[tail_at] = Codec<D>::narrow(Codec<S>::widen(tail_raw));
    } else if (has_edges(w)) {
      cast_edges<S, D, T, U>(d, s, c.chunk, g);
    }
  }
}

// ---- publish ------------------------------------------------------------------------------
// One rank's accumulations at the end of a minibatch: acc[i] /= divisor in place (a correctly
// rounded IEEE division, rounded to the accumulation dtype) and out[i] = narrow_O(acc[i]).
template <class A, class O>
__global__ __launch_bounds__(kThreads) void publish_kernel(const PublishLaunch launch) {
  typedef typename Codec<A>::raw_t araw_t;
  typedef typename Codec<O>::raw_t oraw_t;
  typedef typename Quad<A>::vec_t avec_t;
  typedef typename Quad<O>::vec_t ovec_t;
  const uint32_t tid = threadIdx.x;
  TileCursor cur;
  PublishDesc it = {};
  for (uint32_t t = blockIdx.x; t < launch.tt.n_tiles; t += gridDim.x) {
    if (!cursor_holds(cur, t)) {
      cursor_seek(launch.tt, t, cur);
      it = launch.item[cur.item];  // issued together with the loads of cursor_enter
      cursor_enter(launch.tt, cur);
    }
    const TileCoord c = cursor_coord(launch.tt, cur, t);
    const uint64_t seg = it.seg_elems;
    const uint64_t in_seg = (uint64_t)c.chunk * kTileElems;
    araw_t* acc = reinterpret_cast<araw_t*>(launch.region + it.acc_off) + in_seg;
    oraw_t* out = it.out ? reinterpret_cast<oraw_t*>(it.out) + in_seg : nullptr;
    const uint64_t left = seg - in_seg;
    if (left >= kTileElems && (((uintptr_t)acc) & (sizeof(avec_t) - 1)) == 0 &&
        (((uintptr_t)out) & (sizeof(ovec_t) - 1)) == 0) {
      avec_t* ap = reinterpret_cast<avec_t*>(acc) + tid;
      ovec_t* op = reinterpret_cast<ovec_t*>(out) + tid;
      avec_t raw[kUnroll];
      ovec_t cast[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) raw[u] = __builtin_nontemporal_load(ap + u * kThreads);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        float f[4];
        Quad<A>::widen(raw[u], f);
        if (launch.divide) {
          if (launch.divide == 2) {
#pragma unroll
            for (int k = 0; k < 4; ++k) f[k] = f[k] * launch.reciprocal;
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) f[k] = f[k] / launch.divisor;
          }
          raw[u] = Quad<A>::narrow(f);
          Quad<A>::widen(raw[u], f);  // the copy is a cast of the ROUNDED accumulation
        }
        cast[u] = Quad<O>::narrow(f);
      }
      // The two written streams go out one after the other, not interleaved vector by vector
      // (measured: +6..12 %; plain instead of nontemporal stores for the copy change nothing then).
      if (launch.divide) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(raw[u], ap + u * kThreads);
      }
      if (out) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(cast[u], op + u * kThreads);
      }
    } else {
      // element by element (a partial or unaligned tile), all loads before the first store
      constexpr int kPerLane = kTileElems / kThreads;
      const uint32_t n = left < kTileElems ? (uint32_t)left : kTileElems;
      araw_t raw[kPerLane];
#pragma unroll
      for (int j = 0; j < kPerLane; ++j)
        if (j * kThreads + tid < n) raw[j] = acc[j * kThreads + tid];
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        const uint32_t i = j * kThreads + tid;
        if (i < n) {
          if (launch.divide) {
            const float x = Codec<A>::widen(raw[j]);
            raw[j] = Codec<A>::narrow(launch.divide == 2 ? x * launch.reciprocal : x / launch.divisor);
            acc[i] = raw[j];
          }
          if (out) out[i] = Codec<O>::narrow(Codec<A>::widen(raw[j]));
        }
      }
    }
  }
}

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
  void* allocation = nullptr;  // the hipMalloc (null without backing)
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
    ODC_HIP_TRY(hipGetDevice(&prev_));
    if (prev_ != device) {
      ODC_HIP_TRY(hipSetDevice(device));
      switched_ = true;
    }
    return ODC_OK;
  }
  ~DeviceGuard() {
    if (switched_) (void)hipSetDevice(prev_);
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

// The one place kernels are launched from. On a dry-run arena the launch is only counted: the
// host-side validation, work-list splitting and tile tables have all run by then.
template <class Launch>
int launch_tiles(const odc_arena* a, void (*kernel)(const Launch), uint32_t grid, uint32_t lds_bytes, void* stream,
                 const Launch& L, uint32_t threads = kThreads) {
  if (grid == 0 || grid > L.tt.n_tiles || L.tt.n_tiles != L.tt.tiles_per_rank * L.tt.world)
    return fail(ODC_ERR_INVALID, "internal: launch of %u workgroups over %u tiles", grid, L.tt.n_tiles);
  if (a->dry_run) {
    g_dry_launches += 1;
    g_dry_tiles += L.tt.n_tiles;
    g_dry_workgroups += grid;
    return ODC_OK;
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds_bytes, static_cast<hipStream_t>(stream), L);
  ODC_HIP_TRY(hipGetLastError());
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
  if (a->rank_stride > (~0ull) / world_size) {
    delete a;
    return fail(ODC_ERR_INVALID, "arena size overflows 64 bits");
  }
  if (!(flags & ODC_ARENA_NO_BACKING)) {
    hipError_t e = hipGetDevice(&a->device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&a->n_cu, hipDeviceAttributeMultiprocessorCount, a->device);
    if (e == hipSuccess) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, a->device) == hipSuccess && v > 0)
        a->lds_per_cu = v;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, a->device) == hipSuccess && v > 0)
        a->lds_per_wg_max = v;
      (void)hipGetLastError();
    }
    // hipMalloc promises 256 B alignment only; the regions shall start on stride_align boundaries
    void* p = nullptr;
    const uint64_t slack = stride_align > kAlign ? stride_align : 0;
    if (e == hipSuccess) e = hipMalloc(&p, a->rank_stride * world_size + slack);
    if (e != hipSuccess) {
      delete a;
      return fail(e == hipErrorOutOfMemory ? ODC_ERR_NOMEM : ODC_ERR_HIP,
                  "creating a %u x %llu byte arena failed: %s", world_size,
                  (unsigned long long)bytes_per_rank, hipGetErrorString(e));
    }
    a->allocation = p;
    a->base = reinterpret_cast<uint8_t*>(round_up((uint64_t)(uintptr_t)p, stride_align));
    a->origin = a->base;
    if (a->n_cu <= 0) a->n_cu = 256;
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
    hipError_t e = hipGetDevice(&cur);
    if (e == hipSuccess && cur != a->device) e = hipSetDevice(a->device);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipFree(a->allocation);
    if (e != hipSuccess) rc = fail(ODC_ERR_HIP, "releasing the arena failed: %s", hipGetErrorString(e));
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
template <class Units, class Take>
int fill_launch(TileTable& tt, uint32_t world, uint32_t n_items, uint32_t* next, uint64_t tile_units,
                Units units, Take take) {
  const int n = fill_tile_table(tt, world, n_items, next, tile_units, units, take);
  if (n < 0)
    return fail(ODC_ERR_INVALID, "item %d: %llu units per rank is too large for one launch", -1 - n,
                (unsigned long long)units((uint32_t)(-1 - n)));
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

typedef void (*accum_fn)(const AccumLaunch);
typedef void (*cast_gather_fn)(const CastGatherLaunch);
typedef void (*publish_fn)(const PublishLaunch);

#define ODC_FOR_EACH_DTYPE_PAIR(X)                    \
  X(ODC_DTYPE_BF16, bf16_tag, ODC_DTYPE_BF16, bf16_tag) \
  X(ODC_DTYPE_BF16, bf16_tag, ODC_DTYPE_F16, f16_tag)   \
  X(ODC_DTYPE_BF16, bf16_tag, ODC_DTYPE_F32, f32_tag)   \
  X(ODC_DTYPE_F16, f16_tag, ODC_DTYPE_BF16, bf16_tag)   \
  X(ODC_DTYPE_F16, f16_tag, ODC_DTYPE_F16, f16_tag)     \
  X(ODC_DTYPE_F16, f16_tag, ODC_DTYPE_F32, f32_tag)     \
  X(ODC_DTYPE_F32, f32_tag, ODC_DTYPE_BF16, bf16_tag)   \
  X(ODC_DTYPE_F32, f32_tag, ODC_DTYPE_F16, f16_tag)     \
  X(ODC_DTYPE_F32, f32_tag, ODC_DTYPE_F32, f32_tag)

accum_fn pick_accum(int g, int a, bool store) {  // (gradient dtype, accumulation dtype)
#define X(E1, T1, E2, T2) \
  if (g == E1 && a == E2)                                                            \
    return store ? accum_kernel<T1, T2, true, kStoreThreads, kStoreUnroll> : accum_kernel<T1, T2, false, kThreads, kUnroll>;
  ODC_FOR_EACH_DTYPE_PAIR(X)
#undef X
  return nullptr;
}

cast_gather_fn pick_cast_gather(int s, int d) {  // (shard dtype, output dtype)
#define X(E1, T1, E2, T2) if (s == E1 && d == E2) return cast_gather_kernel<T1, T2, kCopyThreads, kCopyUnroll>;
  ODC_FOR_EACH_DTYPE_PAIR(X)
#undef X
  return nullptr;
}

publish_fn pick_publish(int a, int o) {  // (accumulation dtype, output dtype)
#define X(E1, T1, E2, T2) if (a == E1 && o == E2) return publish_kernel<T1, T2>;
  ODC_FOR_EACH_DTYPE_PAIR(X)
#undef X
  return nullptr;
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
    if (int rc = launch_tiles(a, gather_kernel<kCopyThreads, kCopyUnroll>, grid,
                              lds_claim_for(a, opt.gather_resident_cap, grid, L.tt.n_tiles), stream, L, kCopyThreads))
      return rc;
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
  const cast_gather_fn kernel = pick_cast_gather(src_dtype, dst_dtype);
  if (!kernel) return fail(ODC_ERR_UNSUPPORTED, "gather from dtype %d into dtype %d is not implemented", src_dtype, dst_dtype);
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
          L.item[slot] = {static_cast<uint8_t*>(items[i].dst), items[i].src_offset, items[i].shard_elems};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    const uint32_t grid = grid_for(a, opt.gather_blocks_per_cu, L.tt.n_tiles);
    if (int rc = launch_tiles(a, kernel, grid, lds_claim_for(a, opt.cast_resident_cap, grid, L.tt.n_tiles), stream, L,
                              kCopyThreads))
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
    L.tt.order = kRanksInterleaved;  // a write-only stream runs fastest with the ranks interleaved
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, a->world, n_spans, &next, kTileBytes, [&](uint32_t i) { return spans[i].nbytes; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {spans[i].offset, spans[i].nbytes};
        });
    if (n < 0) return n;
    if (n == 0) continue;
    const uint32_t grid = grid_for(a, opt.clear_blocks_per_cu, L.tt.n_tiles);
    if (int rc = launch_tiles(a, clear_kernel, grid, 0u, stream, L)) return rc;
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
  const accum_fn kernel = pick_accum(grad_dtype, acc_dtype, store);
  if (!kernel)
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
  uint32_t next = 0;
  while (next < n_items) {
    AccumLaunch L;
    L.base = a->origin;
    L.rank_stride = a->rank_stride;
    L.tt.order = (uint32_t)opt.rank_major;
    L.tt.first_rank = 0;
    const int n = fill_launch(
        L.tt, a->world, n_items, &next, kTileElems, [&](uint32_t i) { return items[i].shard_elems; },
        [&](uint32_t slot, uint32_t i) {
          L.item[slot] = {static_cast<const uint8_t*>(items[i].grad), items[i].grad_elems, items[i].acc_offset,
                          items[i].shard_elems};
        });
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
    // Launch shape. With tile-aligned rank regions and buffers, one workgroup per tile streams
    // fastest down to segments of a few hundred tiles (measured: +1.0..2.3 % over the persistent
    // shape at W=4..32). The persistent shape, one workgroup per CU, wins on shorter segments
    // (+1.6 % at W=64, 92 tiles per segment; level at W=128), but only while every rank's chunk of
    // the gradient and of the accumulation starts on a 128 B line: with nothing else resident to
    // cover for it, a workgroup whose wavefronts straddle lines, or that meets heads, tails and
    // padding, falls behind (measured: -7 % on 16 B aligned uneven shards). So: ragged launches
    // and all but the shortest segments run one workgroup per tile.
    // (Measured for 16-bit gradients into fp32 accumulations; fp32 gradients, 12 B per element,
    // run 2 % faster one workgroup per tile.)
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
    if (int rc = launch_tiles(a, kernel, grid, lds_claim_for(a, cap, grid, L.tt.n_tiles), stream, L,
                              store ? kStoreThreads : kThreads))
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
  const publish_fn kernel = pick_publish(acc_dtype, out_dtype);
  if (!kernel) return fail(ODC_ERR_UNSUPPORTED, "publish from dtype %d into dtype %d is not implemented", acc_dtype, out_dtype);
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
    if (int rc = launch_tiles(a, kernel, grid, lds_claim_for(a, opt.publish_resident_cap, grid, L.tt.n_tiles), stream, L))
      return rc;
  }
  return ODC_OK;
}

}  // extern "C"
