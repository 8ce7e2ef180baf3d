// odc_kernels.hip — the device side of libodc_hip.so for gfx950 (MI355X, CDNA4): the kernels and
// the few HIP runtime calls behind namespace odc_device (odc_launch.h). The C ABI, the symmetric
// arena, validation and launch planning are in odc_host.cpp.
//
// Five streaming kernels, all HBM-bandwidth bound (no MFMA, no LDS):
//   gather_kernel       : W shard regions -> one flat buffer          (read 1 B + write 1 B per byte)
//   cast_gather_kernel  : the same with a dtype conversion on the way (fp32 -> bf16: 6 B per element),
//                         into one buffer or into every rank's own region (the conversion pass)
//   accum_kernel        : acc_r += widen(grad chunk r), in place      (bf16 -> fp32: 10 B per element)
//                         or acc_r = +0 + widen(grad chunk r), acc not read          (6 B per element)
//   clear_kernel        : zero a span in every rank region            (write 1 B per byte)
//   publish_kernel      : one rank's acc /= divisor, plus a cast copy (end of a minibatch)
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

#include "odc_hip.h"
#include "odc_launch.h"
#include "odc_tiles.h"

namespace {

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

// ------------------------------------------------------------------------------------------------
// device side
// ------------------------------------------------------------------------------------------------
using namespace odc_tiles;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

using namespace odc_launch;

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
// dst[r*stride + i] = narrow_D(widen_S(region_r[off + i])): the gather of shards kept in one dtype
// (fp32 master copies) into a full parameter of another (bf16), in one pass (stride = the
// segment's size: the converted segments lie back to back), or, with stride = the distance
// between rank regions and dst inside rank 0's region, the conversion of every rank's shard into
// a second symmetric buffer.
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
    uint8_t* d = it.dst + (uint64_t)c.rank * it.dst_stride;
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
// dtype dispatch
// ------------------------------------------------------------------------------------------------
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

// The launch's own status, not hipGetLastError(): that one also reports what an earlier,
// unrelated HIP call of the same host thread left behind.
template <class Launch>
int launch(void (*kernel)(const Launch), const Launch& L, uint32_t grid, uint32_t threads, uint32_t lds_bytes,
           void* stream) {
  if (!kernel) return (int)hipErrorInvalidDeviceFunction;
  void* args[] = {const_cast<Launch*>(&L)};
  return (int)hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(threads), args, lds_bytes,
                              static_cast<hipStream_t>(stream));
}

}  // namespace

// ------------------------------------------------------------------------------------------------
// namespace odc_device (odc_launch.h)
// ------------------------------------------------------------------------------------------------
namespace odc_device {

int get_current(int* device) { return (int)hipGetDevice(device); }

int set_current(int device) { return (int)hipSetDevice(device); }

int properties(int device, Properties* out) {
  hipError_t e = hipDeviceGetAttribute(&out->n_cu, hipDeviceAttributeMultiprocessorCount, device);
  if (e != hipSuccess) return (int)e;
  if (out->n_cu <= 0) out->n_cu = 256;
  // the two LDS sizes only matter for residency caps: keep the gfx950 values when a query fails
  out->lds_per_cu = 160 * 1024;
  out->lds_per_wg_max = 64 * 1024;
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device) == hipSuccess && v > 0)
    out->lds_per_cu = v;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, device) == hipSuccess && v > 0)
    out->lds_per_wg_max = v;
  (void)hipGetLastError();
  return 0;
}

int allocate(void** ptr, uint64_t bytes) { return (int)hipMalloc(ptr, bytes); }

int release(void* ptr) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipFree(ptr);
  return (int)e;
}

bool is_out_of_memory(int code) { return code == (int)hipErrorOutOfMemory; }

const char* error_string(int code) { return hipGetErrorString(static_cast<hipError_t>(code)); }

bool has_accum(int g, int a) { return pick_accum(g, a, false) != nullptr; }
bool has_cast_gather(int s, int d) { return pick_cast_gather(s, d) != nullptr; }
bool has_publish(int a, int o) { return pick_publish(a, o) != nullptr; }

int launch_gather(const GatherLaunch& L, uint32_t grid, uint32_t lds_bytes, void* stream) {
  return launch(gather_kernel<kCopyThreads, kCopyUnroll>, L, grid, kCopyThreads, lds_bytes, stream);
}

int launch_cast_gather(int s, int d, const CastGatherLaunch& L, uint32_t grid, uint32_t lds_bytes, void* stream) {
  return launch(pick_cast_gather(s, d), L, grid, kCopyThreads, lds_bytes, stream);
}

int launch_accum(int g, int a, bool store, const AccumLaunch& L, uint32_t grid, uint32_t lds_bytes, void* stream) {
  return launch(pick_accum(g, a, store), L, grid, store ? kStoreThreads : kThreads, lds_bytes, stream);
}

int launch_clear(const ClearLaunch& L, uint32_t grid, void* stream) {
  return launch(clear_kernel, L, grid, kThreads, 0u, stream);
}

int launch_publish(int a, int o, const PublishLaunch& L, uint32_t grid, uint32_t lds_bytes, void* stream) {
  return launch(pick_publish(a, o), L, grid, kThreads, lds_bytes, stream);
}

}  // namespace odc_device
