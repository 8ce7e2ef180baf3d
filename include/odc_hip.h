/*
 * odc_hip.h — C ABI of libodc_hip.so, the MI355X (gfx950) native layer under the ODC
 * data-parallel primitives: gather (W sharded params -> one full flat param) and
 * scatter-accumulate (full gradients added into W per-shard accumulation buffers).
 *
 * It replaces, for one GPU holding W "virtual ranks", what the reference gets from
 *   - csrc/tensor_ipc/tensor_ipc.cu:24-57 + binding.cpp:8-11  (peer memory handles),
 *   - nvshmem.core.tensor / get_peer_tensor as used by odc/primitives/utils.py:52-75,
 *   - the ATen copy_/add_/fill_ calls on the hot path
 *     (odc/primitives/gather.py:121-127, scatter_accumulate.py:386,585-587,666-669).
 *
 * Conventions
 *   - Every function returns ODC_OK (0) or a negative odc_status; nothing aborts the process
 *     (the reference's native code prints and exit(1)s: tensor_ipc.cu:5-22).
 *     odc_last_error() returns a thread-local, human-readable message for the last failure.
 *   - All launches are asynchronous on the hipStream_t passed as `stream` (NULL = the null
 *     stream); no entry point synchronises the host except odc_arena_destroy.
 *   - Callable from any host thread; the arena's device is made current for the call.
 *   - Pointers are plain device pointers; sizes are bytes unless the name says `elems`.
 */
#ifndef ODC_HIP_H_
#define ODC_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ODC_HIP_ABI_VERSION 3

typedef enum odc_status {
  ODC_OK = 0,
  ODC_ERR_INVALID = -1,     /* bad argument (null, zero world size, misaligned offset, ...) */
  ODC_ERR_NOMEM = -2,       /* symmetric arena exhausted */
  ODC_ERR_HIP = -3,         /* a HIP runtime call failed (message carries hipGetErrorString) */
  ODC_ERR_UNSUPPORTED = -4, /* dtype combination not implemented */
  ODC_ERR_NOT_FOUND = -5,   /* offset / pointer does not name a live allocation */
  ODC_ERR_NO_BACKING = -6   /* compute requested on a bookkeeping-only arena */
} odc_status;

typedef enum odc_dtype {
  ODC_DTYPE_BF16 = 0,
  ODC_DTYPE_F16 = 1,
  ODC_DTYPE_F32 = 2
} odc_dtype;

/* ------------------------------------------------------------------------------------------
 * Symmetric arena: ONE hipMalloc carved into `world_size` rank regions. An allocation returns a
 * single byte offset that is valid in every rank region, which is the property the reference
 * gets from the NVSHMEM symmetric heap (odc/primitives/utils.py:52-75,126-143).
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_arena odc_arena;

enum {
  ODC_ARENA_DEVICE = 0,     /* hipMalloc-backed (the product path) */
  ODC_ARENA_NO_BACKING = 1, /* offsets only, no memory: for sizing an arena before creating it.
                               Every compute entry point refuses it with ODC_ERR_NO_BACKING. */
  ODC_ARENA_DRY_RUN = 2     /* no memory and no GPU needed: the compute entry points validate their
                               arguments, split the work list and plan every launch against a
                               fictitious base address, then count the launch instead of issuing it
                               (odc_get_option "dry_run_launches" / "dry_run_tiles" /
                               "dry_run_workgroups"; odc_set_option("dry_run_reset", 0) zeroes them).
                               For testing the host side of the library without a device; implies
                               ODC_ARENA_NO_BACKING for odc_arena_ptr / odc_arena_locate. */
};

typedef struct odc_arena_info {
  uint32_t world_size;
  int32_t device;           /* HIP device ordinal, -1 for a bookkeeping-only arena */
  uint32_t flags;
  uint32_t n_allocations;   /* live allocations */
  uint64_t bytes_per_rank;  /* usable bytes in each rank region */
  uint64_t rank_stride;     /* distance in bytes between consecutive rank regions */
  uint64_t base;            /* device address of rank 0's region (0 without backing) */
  uint64_t bytes_in_use;    /* per rank, live allocations incl. alignment rounding */
  uint64_t high_water;      /* per rank, highest offset ever handed out */
} odc_arena_info;

/* Create an arena of world_size regions of bytes_per_rank bytes each (at most 2^60) on the
 * current device.
 * Replaces nvshmem.core.init + NVSHMEM_SYMMETRIC_SIZE (utils.py:18-49, launch.sh:135). */
int odc_arena_create(uint32_t world_size, uint64_t bytes_per_rank, uint32_t flags,
                     odc_arena** out);

/* Synchronise the device and release the arena. Replaces nvshmem.core.finalize (utils.py:84-85). */
int odc_arena_destroy(odc_arena* arena);

/* Symmetric allocation of nbytes (rounded up to 256 B) in every rank region. *offset is a
 * multiple of 256; for allocations of 16 KiB (one kernel tile) or more it is a multiple of 16 KiB,
 * and rank regions are that far apart or a multiple of it, so the buffer starts on a tile boundary
 * in every region: the read-modify-write of the scatter-accumulate is up to 5.5 % slower on
 * accumulations that do not (options "alloc_align" / "rank_stride_align"). Replaces
 * nvshmem.core.tensor (utils.py:52-56). */
int odc_arena_alloc(odc_arena* arena, uint64_t nbytes, uint64_t* offset);

/* Release one allocation by its offset. Replaces nvshmem.core.free_tensor (utils.py:78-81). */
int odc_arena_free(odc_arena* arena, uint64_t offset);

/* Drop every allocation (registry finalize, utils.py:163-169). */
int odc_arena_reset(odc_arena* arena);

int odc_arena_get_info(const odc_arena* arena, odc_arena_info* info);

/* Device address of `offset` inside rank `rank`'s region; NULL on a bad rank/offset or without
 * backing. Replaces nvshmem.core.get_peer_tensor (utils.py:61-75) and
 * tensor_ipc.reconstruct_tensor (tensor_ipc.cu:46-57). */
void* odc_arena_ptr(const odc_arena* arena, uint32_t rank, uint64_t offset);

/* Reverse lookup: which rank region and which allocation holds device address `ptr`
 * (the registry's data_ptr -> key map, utils.py:139,158-161, and the base/offset split of
 * tensor_ipc.get_ipc_handle, tensor_ipc.cu:24-44). alloc_offset is the start of the allocation,
 * inner the distance of ptr from it. Any out pointer may be NULL. */
int odc_arena_locate(const odc_arena* arena, const void* ptr, uint32_t* rank,
                     uint64_t* alloc_offset, uint64_t* inner);

/* ------------------------------------------------------------------------------------------
 * gather — for every item and every rank r:
 *     dst[r*shard_bytes : (r+1)*shard_bytes] = rank r's bytes [src_offset, src_offset+shard_bytes)
 * i.e. output.view(W,-1)[r].copy_(peer_tensors[r])  (odc/primitives/gather.py:116-127).
 * All items go out in as few launches as possible (one per ODC_MAX_ITEMS_PER_LAUNCH items); a
 * byte copy, so any element type. first_rank rotates the order in which rank regions are walked
 * (gather.py:122); it never changes the result. dst must not overlap the arena ranges read.
 * ---------------------------------------------------------------------------------------- */
#define ODC_MAX_ITEMS_PER_LAUNCH 64

typedef struct odc_gather_item {
  void* dst;             /* device pointer to W*shard_bytes writable bytes */
  uint64_t src_offset;   /* symmetric byte offset of the shard in each rank region */
  uint64_t shard_bytes;  /* bytes contributed by each rank (may be 0) */
} odc_gather_item;

int odc_gather(odc_arena* arena, const odc_gather_item* items, uint32_t n_items,
               uint32_t first_rank, void* stream);

/* ------------------------------------------------------------------------------------------
 * gather with cast — the same as gather, but shards of src_dtype are converted to dst_dtype on
 * the way (exact widening, round-to-nearest-even narrowing):
 *     dst[r*shard_elems + i] = cast(rank r's element i at src_offset)
 * One pass instead of the reference's gather in the shard dtype followed by a cast of the full
 * parameter (odc/fsdp/fsdp1.py:199-223, odc/fsdp/fsdp2.py:341-343).
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_gather_cast_item {
  void* dst;             /* device pointer to W*shard_elems elements of dst_dtype */
  uint64_t src_offset;   /* symmetric byte offset of the shard, src_dtype aligned */
  uint64_t shard_elems;  /* elements contributed by each rank */
} odc_gather_cast_item;

int odc_gather_cast(odc_arena* arena, const odc_gather_cast_item* items, uint32_t n_items,
                    int src_dtype, int dst_dtype, uint32_t first_rank, void* stream);

/* ------------------------------------------------------------------------------------------
 * convert — for every item and EVERY rank r, inside r's own region:
 *     region_r[dst_offset ...][i] = cast(region_r[src_offset ...][i])      for i < elems
 * (exact widening, round-to-nearest-even narrowing; equal dtypes make it a symmetric copy): one
 * symmetric buffer converted into another in one launch over all ranks. It keeps a copy of the
 * sharded parameters in the compute dtype, so that the gathers of a minibatch move 2 + 2 bytes
 * per element instead of converting on the way: the low-precision shard that the reference's
 * FSDP1 path copies once until flush() (odc/primitives/utils.py:103-116, odc/fsdp/fsdp1.py:239-247;
 * there every process converts its own shard, here one launch does all W). Source and
 * destination of an item must not overlap.
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_convert_item {
  uint64_t src_offset;   /* symmetric byte offset of the source, src_dtype aligned */
  uint64_t dst_offset;   /* symmetric byte offset of the destination, dst_dtype aligned */
  uint64_t elems;        /* elements converted per rank */
} odc_convert_item;

int odc_convert(odc_arena* arena, const odc_convert_item* items, uint32_t n_items, int src_dtype,
                int dst_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * scatter-accumulate — for every item and every rank r, with g = the item's gradient viewed as
 * W consecutive chunks of shard_elems elements (elements at index >= grad_elems read as +0):
 *     acc_r[0:shard_elems] += g[r*shard_elems : (r+1)*shard_elems]
 * where acc_r is rank r's region at acc_offset. One IEEE add per element in fp32 after exact
 * widening, rounded to acc_dtype with round-to-nearest-even when acc_dtype is 16 bit. This is
 * acc[start:start+size].add_(buf[:size]) over all sub-buffers (scatter_accumulate.py:381-391)
 * fused with the staging copies (scatter_accumulate.py:649-669); the zero tail is the F.pad of
 * odc/fsdp/fsdp1.py:25-38. The items of one call must not overlap each other in the accumulations
 * (they are worked on concurrently, in an order of the library's choosing: items of less than one
 * tile per rank go last).
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_accum_item {
  const void* grad;      /* device pointer to the full gradient, grad_dtype */
  uint64_t grad_elems;   /* valid elements at grad, <= W*shard_elems */
  uint64_t acc_offset;   /* symmetric byte offset of the accumulation slice, acc_dtype aligned */
  uint64_t shard_elems;  /* elements accumulated per rank */
} odc_accum_item;

int odc_scatter_accumulate(odc_arena* arena, const odc_accum_item* items, uint32_t n_items,
                           int grad_dtype, int acc_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * scatter-store — the first scatter-accumulate after a clear, without the clear: for every item
 * and every rank r
 *     acc_r[0:shard_elems] = (+0) + g[r*shard_elems : (r+1)*shard_elems]
 * i.e. exactly the bits that acc.fill_(0) (scatter_accumulate.py:585-587) followed by
 * acc.add_(buf) (scatter_accumulate.py:386) leaves (a -0 gradient becomes +0, padding becomes
 * +0), in one pass that never reads the accumulation: 6 instead of 4 + 10 bytes per element
 * for bf16 gradients and fp32 accumulations. Same items, dtypes and checks as
 * odc_scatter_accumulate. The items of one call must not overlap each other.
 * ---------------------------------------------------------------------------------------- */
int odc_scatter_store(odc_arena* arena, const odc_accum_item* items, uint32_t n_items,
                      int grad_dtype, int acc_dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * clear — zero bytes [offset, offset+nbytes) in every rank region, for every span, in one
 * launch per ODC_MAX_ITEMS_PER_LAUNCH spans (a fill kernel, safe to capture in a HIP graph).
 * Replaces acc.fill_(0) per key (scatter_accumulate.py:585-587).
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_span {
  uint64_t offset;
  uint64_t nbytes;
} odc_span;

int odc_clear(odc_arena* arena, const odc_span* spans, uint32_t n_spans, void* stream);

/* ------------------------------------------------------------------------------------------
 * publish — end-of-minibatch pass over ONE rank's accumulations, for every item:
 *     acc[i] = acc[i] / divisor        (in place, correctly rounded; skipped when divisor == 1)
 *     out[i] = cast_to_out_dtype(acc[i])                      (skipped when out is NULL)
 * Replaces `acc /= W` / `_div_if_needed(acc, factor)` followed by `acc.to(param_dtype)`
 * (odc/fsdp/fsdp1.py:324-335, odc/fsdp/fsdp2.py:846-847,897-899) with one read of the shard.
 * ---------------------------------------------------------------------------------------- */
typedef struct odc_publish_item {
  uint64_t acc_offset;   /* symmetric byte offset of the accumulation (slice), acc_dtype aligned */
  uint64_t elems;
  void* out;             /* device pointer to elems elements of out_dtype, or NULL */
} odc_publish_item;

int odc_publish(odc_arena* arena, uint32_t rank, const odc_publish_item* items, uint32_t n_items,
                int acc_dtype, int out_dtype, float divisor, void* stream);

/* ------------------------------------------------------------------------------------------
 * Library-wide
 * ---------------------------------------------------------------------------------------- */
const char* odc_last_error(void);
int odc_abi_version(void);

/* Launch-shape knobs, for measurement.
 *  - "gather_blocks_per_cu", "accum_blocks_per_cu", "store_blocks_per_cu", "clear_blocks_per_cu",
 *    "publish_blocks_per_cu": persistent workgroups per CU walking the tiles with a grid-stride
 *    loop; 0 = one workgroup per tile, dealt out by the hardware dispatcher. accum_blocks_per_cu
 *    defaults to -1: one per tile, except 1 persistent per CU when the launch's segments average
 *    fewer than "accum_persistent_below_tiles" tiles (default 0: never).
 *  - "gather_resident_cap", "cast_resident_cap", "accum_resident_cap", "store_resident_cap",
 *    "publish_resident_cap": for one-workgroup-per-tile launches, the most workgroups resident per
 *    CU (enforced by claiming unused LDS; 0 = no cap, no claim; all default to 0).
 *  - "rank_major" (gather) and "accum_tile_order" (scatter-accumulate, scatter-store): 1 = walk a
 *    rank's whole shard before the next rank, item by item; 0 = interleave ranks tile by tile;
 *    2 = rank outermost: all items' segments of rank 0, then of rank 1, ... accum_tile_order 3,
 *    its default, picks 2 when segments average fewer than "accum_short_segment_tiles" (256)
 *    tiles and 1 otherwise.
 *  - "accum_small_items_last" (default 1): scatter-accumulate and scatter-store launch the items
 *    of less than one tile per rank after the others; 0 keeps the caller's order.
 *  - "rank_stagger_bytes" (extra distance between rank regions), "rank_stride_align" (rank regions
 *    start on multiples of it, default 16384 = one tile) and "alloc_align" (allocations of at
 *    least this many bytes start on multiples of it, default 16384; smaller ones on 256): read
 *    when an arena is created and rounded up to multiples of 256; at most 2^40 each.
 * Unknown names return ODC_ERR_INVALID. Results never depend on these. */
int odc_set_option(const char* name, int64_t value);
int odc_get_option(const char* name, int64_t* value);

#ifdef __cplusplus
}
#endif

#endif /* ODC_HIP_H_ */
