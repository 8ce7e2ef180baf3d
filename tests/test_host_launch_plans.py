"""The host side of every compute entry point, exercised WITHOUT a GPU on a dry-run arena
(ODC_ARENA_DRY_RUN): argument validation, the split of long item lists over launches, tile counts
and launch shapes. Nothing is launched; the library counts what it would have launched.

A host-side bug here (an item list cut wrongly, a table that does not add up, a recursion) would
otherwise show only on the GPU box."""

import ctypes
import math

import pytest

from odc_amd import _native

TILE_BYTES = 16 * 1024
TILE_ELEMS = 4096
N_CU = 256  # what a dry-run arena assumes


class DryArena:
    def __init__(self, world, bytes_per_rank):
        self.lib = _native.load()
        self.handle = ctypes.c_void_p()
        _native.check(self.lib.odc_arena_create(world, bytes_per_rank, _native.ODC_ARENA_DRY_RUN, ctypes.byref(self.handle)))
        self.world = world
        info = _native.ArenaInfo()
        _native.check(self.lib.odc_arena_get_info(self.handle, ctypes.byref(info)))
        self.info = info
        _native.set_option("dry_run_reset", 0)

    def counters(self):
        return tuple(_native.get_option(n) for n in ("dry_run_launches", "dry_run_tiles", "dry_run_workgroups"))

    def close(self):
        _native.check(self.lib.odc_arena_destroy(self.handle))


@pytest.fixture
def arena():
    made = []

    def _make(world, bytes_per_rank=1 << 30):
        a = DryArena(world, bytes_per_rank)
        made.append(a)
        return a

    yield _make
    for a in made:
        a.close()


OUTSIDE = 1 << 33  # a "device address" far from the dry-run arena's fictitious base (1 << 44)
FAR_OUTSIDE = 1 << 50  # the same, above the arena: room for outputs of 2^46 bytes


def test_dry_run_arena_has_no_memory_but_plans(arena):
    a = arena(8)
    assert a.info.device == -1 and a.info.base == 0 and a.info.flags & _native.ODC_ARENA_NO_BACKING
    assert not a.lib.odc_arena_ptr(a.handle, 0, 0)  # no memory to point at
    off = ctypes.c_uint64()
    _native.check(a.lib.odc_arena_alloc(a.handle, 1 << 20, ctypes.byref(off)))
    items = (_native.GatherItem * 1)(_native.GatherItem(OUTSIDE, off.value, 1 << 20))
    _native.check(a.lib.odc_gather(a.handle, items, 1, 0, None))
    assert a.counters() == (1, 8 * 64, 8 * 64)  # one launch, one workgroup per 16 KiB tile per rank


def test_a_plain_no_backing_arena_still_refuses_compute():
    lib = _native.load()
    handle = ctypes.c_void_p()
    _native.check(lib.odc_arena_create(4, 1 << 20, _native.ODC_ARENA_NO_BACKING, ctypes.byref(handle)))
    items = (_native.GatherItem * 1)(_native.GatherItem(OUTSIDE, 0, 4096))
    assert lib.odc_gather(handle, items, 1, 0, None) == _native.ODC_ERR_NO_BACKING
    _native.check(lib.odc_arena_destroy(handle))


@pytest.mark.parametrize("n_items", [1, 9, 63, 64, 65, 128, 129, 300])
def test_long_item_lists_are_split_over_launches(arena, n_items):
    W = 4
    a = arena(W)
    sizes = [(7 * i) % 5 * 10_000 + (i % 3) * 17 for i in range(n_items)]  # some are empty
    items = (_native.GatherItem * n_items)()
    off = 0
    for it, sz in zip(items, sizes):
        it.dst, it.src_offset, it.shard_bytes = OUTSIDE + 64 * off, off, sz
        off += sz
    _native.check(a.lib.odc_gather(a.handle, items, n_items, W - 1, None))
    nonempty = [s for s in sizes if s]
    launches, tiles, workgroups = a.counters()
    assert launches == math.ceil(len(nonempty) / _native.MAX_ITEMS_PER_LAUNCH)
    assert tiles == W * sum(math.ceil(s / TILE_BYTES) for s in nonempty)
    assert workgroups == tiles  # the gather runs one workgroup per tile


def test_accumulate_launch_shapes(arena):
    W = 8
    a = arena(W)
    # line-aligned whole shards in short segments: one workgroup per tile by default; the persistent
    # shape, one workgroup per CU, only when asked for through the threshold
    shard = 1 << 18
    items = (_native.AccumItem * 2)(
        _native.AccumItem(OUTSIDE, W * shard, 0, shard), _native.AccumItem(OUTSIDE + (1 << 30), W * shard, 4 * shard, shard)
    )
    _native.check(a.lib.odc_scatter_accumulate(a.handle, items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
    launches, tiles, workgroups = a.counters()
    assert (launches, tiles, workgroups) == (1, 2 * W * shard // TILE_ELEMS, 2 * W * shard // TILE_ELEMS)
    _native.set_option("dry_run_reset", 0)
    _native.set_option("accum_persistent_below_tiles", 128)  # segments of 64 tiles are below it
    try:
        _native.check(a.lib.odc_scatter_accumulate(a.handle, items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
        assert a.counters() == (1, tiles, N_CU)
        # the same as a store, or with a gradient that ends early (padding): one workgroup per tile
        _native.set_option("dry_run_reset", 0)
        _native.check(a.lib.odc_scatter_store(a.handle, items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
        assert a.counters() == (1, tiles, tiles)
        _native.set_option("dry_run_reset", 0)
        items[1].grad_elems -= 5
        _native.check(a.lib.odc_scatter_accumulate(a.handle, items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
        assert a.counters() == (1, tiles, tiles)
    finally:
        _native.set_option("accum_persistent_below_tiles", 0)
    # long segments (128 tiles and more): one workgroup per tile, unless the knob says otherwise
    _native.set_option("dry_run_reset", 0)
    shard = 1 << 20
    long_items = (_native.AccumItem * 2)(
        _native.AccumItem(OUTSIDE, W * shard, 0, shard), _native.AccumItem(OUTSIDE + (1 << 30), W * shard, 4 * shard, shard)
    )
    _native.check(a.lib.odc_scatter_accumulate(a.handle, long_items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
    long_tiles = 2 * W * shard // TILE_ELEMS
    assert a.counters() == (1, long_tiles, long_tiles)
    _native.set_option("dry_run_reset", 0)
    _native.set_option("accum_blocks_per_cu", 2)
    try:
        _native.check(a.lib.odc_scatter_accumulate(a.handle, long_items, 2, _native.DTYPE_BF16, _native.DTYPE_F32, None))
    finally:
        _native.set_option("accum_blocks_per_cu", -1)
    assert a.counters() == (1, long_tiles, 2 * N_CU)
    # fewer tiles than CUs: the persistent grid shrinks to the tiles
    _native.set_option("dry_run_reset", 0)
    small = (_native.AccumItem * 1)(_native.AccumItem(OUTSIDE, W * 4096, 0, 4096))
    _native.check(a.lib.odc_scatter_accumulate(a.handle, small, 1, _native.DTYPE_BF16, _native.DTYPE_F32, None))
    assert a.counters() == (1, W, W)


def test_clear_cast_gather_and_publish_plan(arena):
    W = 4
    a = arena(W)
    spans = (_native.Span * 3)(_native.Span(0, 100_000), _native.Span(1 << 20, 0), _native.Span(2 << 20, 16_384))
    _native.check(a.lib.odc_clear(a.handle, spans, 3, None))
    assert a.counters() == (1, W * (7 + 1), W * 8)
    _native.set_option("dry_run_reset", 0)
    cast = (_native.GatherCastItem * 1)(_native.GatherCastItem(OUTSIDE, 0, 10_000))
    _native.check(a.lib.odc_gather_cast(a.handle, cast, 1, _native.DTYPE_F32, _native.DTYPE_BF16, 2, None))
    assert a.counters() == (1, W * 3, W * 3)
    _native.set_option("dry_run_reset", 0)
    pub = (_native.PublishItem * 2)(_native.PublishItem(0, 10_000, OUTSIDE), _native.PublishItem(1 << 20, 4096, None))
    _native.check(a.lib.odc_publish(a.handle, 1, pub, 2, _native.DTYPE_F32, _native.DTYPE_BF16, ctypes.c_float(8.0), None))
    assert a.counters() == (1, 3 + 1, 4)  # one rank only


def _error(lib, status):
    assert status != 0
    return status, lib.odc_last_error().decode()


def test_validation_errors_come_back_as_codes_and_messages(arena):
    W = 4
    a = arena(W, 1 << 20)
    lib = a.lib
    G, A = _native.GatherItem, _native.AccumItem
    inside = a.info.bytes_per_rank  # an offset just past the region
    fake_base = 1 << 44

    def gather(*items, first_rank=0):
        arr = (G * len(items))(*items)
        return lib.odc_gather(a.handle, arr, len(items), first_rank, None)

    def accum(*items, g=_native.DTYPE_BF16, acc=_native.DTYPE_F32):
        arr = (A * len(items))(*items)
        return lib.odc_scatter_accumulate(a.handle, arr, len(items), g, acc, None)

    assert _error(lib, gather(G(None, 0, 64)))[0] == _native.ODC_ERR_INVALID  # dst NULL
    code, msg = _error(lib, gather(G(OUTSIDE, inside - 32, 64)))
    assert code == _native.ODC_ERR_INVALID and "rank region" in msg
    assert _error(lib, gather(G(OUTSIDE, 0, 64), first_rank=W))[0] == _native.ODC_ERR_INVALID
    code, msg = _error(lib, gather(G(fake_base + 128, 0, 4096)))  # dst inside the arena range it reads
    assert code == _native.ODC_ERR_INVALID and "overlaps" in msg
    assert gather(G(None, 0, 0)) == 0  # an empty item needs no destination
    assert lib.odc_gather(a.handle, None, 1, 0, None) == _native.ODC_ERR_INVALID
    assert lib.odc_gather(None, None, 0, 0, None) == _native.ODC_ERR_INVALID

    code, msg = _error(lib, accum(A(OUTSIDE, W * 64 + 1, 0, 64)))
    assert code == _native.ODC_ERR_INVALID and "grad_elems" in msg
    assert _error(lib, accum(A(OUTSIDE, 64, 2, 64)))[0] == _native.ODC_ERR_INVALID  # acc_offset not fp32 aligned
    assert _error(lib, accum(A(OUTSIDE + 1, 64, 0, 64)))[0] == _native.ODC_ERR_INVALID  # grad not bf16 aligned
    assert _error(lib, accum(A(None, 64, 0, 64)))[0] == _native.ODC_ERR_INVALID
    assert _error(lib, accum(A(OUTSIDE, 64, 0, 64), g=7))[0] == _native.ODC_ERR_INVALID  # unknown dtype code
    assert _error(lib, accum(A(OUTSIDE, 1, 0, 0)))[0] == _native.ODC_ERR_INVALID  # data for an empty shard
    assert accum(A(OUTSIDE, 0, 0, 64)) == 0  # an all-padding gradient is fine
    pub = (_native.PublishItem * 1)(_native.PublishItem(0, 64, OUTSIDE))
    for bad in (0.0, float("nan")):
        assert lib.odc_publish(a.handle, 0, pub, 1, _native.DTYPE_F32, _native.DTYPE_BF16, ctypes.c_float(bad), None) \
            == _native.ODC_ERR_INVALID
    assert lib.odc_publish(a.handle, W, pub, 1, _native.DTYPE_F32, _native.DTYPE_BF16, ctypes.c_float(2.0), None) \
        == _native.ODC_ERR_INVALID
    assert a.counters() == (1, W, W)  # the one valid, non-empty call above: the padding-only accumulate


def test_an_item_too_large_for_one_launch_is_refused_not_truncated(arena):
    a = arena(1, 1 << 46)
    items = (_native.GatherItem * 1)(_native.GatherItem(FAR_OUTSIDE, 0, 1 << 46))  # 2^32 tiles
    status = a.lib.odc_gather(a.handle, items, 1, 0, None)
    assert status == _native.ODC_ERR_INVALID and "too large for one launch" in a.lib.odc_last_error().decode()
    assert a.counters() == (0, 0, 0)
    # just under the limit it is one launch
    _native.set_option("dry_run_reset", 0)
    items[0].shard_bytes = ((1 << 31) - 1) * TILE_BYTES
    _native.check(a.lib.odc_gather(a.handle, items, 1, 0, None))
    assert a.counters() == (1, (1 << 31) - 1, (1 << 31) - 1)


def test_many_large_items_split_when_the_tile_count_would_overflow(arena):
    a = arena(2, 1 << 46)
    per_item = (1 << 29) * TILE_BYTES  # 2^29 tiles per rank, 2^30 per item
    items = (_native.GatherItem * 3)()
    for i, it in enumerate(items):
        it.dst, it.src_offset, it.shard_bytes = FAR_OUTSIDE, i * per_item, per_item
    _native.check(a.lib.odc_gather(a.handle, items, 3, 0, None))
    launches, tiles, _ = a.counters()
    assert (launches, tiles) == (3, 3 << 30)  # 2^30 + 2^30 would reach 2^31: one item per launch


def test_convert_plans_one_launch_over_all_ranks(arena):
    W = 8
    a = arena(W)
    C = _native.ConvertItem
    items = (C * 3)(C(0, 1 << 24, 1_000_000), C(0, 0, 0), C(1 << 25, 1 << 26, 4096))
    _native.check(a.lib.odc_convert(a.handle, items, 3, _native.DTYPE_F32, _native.DTYPE_BF16, None))
    tiles = W * (math.ceil(1_000_000 / TILE_ELEMS) + 1)
    assert a.counters() == (1, tiles, tiles)  # the empty item takes no part
    lib = a.lib

    def status(src, dst, elems, sd=_native.DTYPE_F32, dd=_native.DTYPE_BF16):
        arr = (C * 1)(C(src, dst, elems))
        return lib.odc_convert(a.handle, arr, 1, sd, dd, None)

    assert _error(lib, status(2, 1 << 24, 64))[0] == _native.ODC_ERR_INVALID  # source not fp32 aligned
    assert _error(lib, status(0, (1 << 24) + 1, 64))[0] == _native.ODC_ERR_INVALID  # destination not bf16 aligned
    code, msg = _error(lib, status(0, 128, 64))  # [0, 256) read, [128, 256) written
    assert code == _native.ODC_ERR_INVALID and "overlaps" in msg
    assert status(0, 256, 64) == 0  # touching ranges are fine
    code, msg = _error(lib, status(0, 1 << 24, 1 << 62))  # elems * 4 would wrap around
    assert code == _native.ODC_ERR_INVALID and "exceed" in msg
    assert _error(lib, status(0, a.info.bytes_per_rank - 64, 64))[0] == _native.ODC_ERR_INVALID  # destination leaves the region
    assert _error(lib, status(0, 1 << 24, 64, sd=9))[0] == _native.ODC_ERR_INVALID
    assert lib.odc_convert(a.handle, None, 2, _native.DTYPE_F32, _native.DTYPE_BF16, None) == _native.ODC_ERR_INVALID
    # equal dtypes: a symmetric copy
    assert status(0, 1 << 24, 4096, sd=_native.DTYPE_BF16, dd=_native.DTYPE_BF16) == 0


def test_arena_size_plus_alignment_slack_cannot_wrap():
    """world * rank_stride can fit 64 bits while the allocation, which is one stride alignment
    larger so that rank 0 can start on a multiple of it, does not: 17 regions of 986 895 * 2^40
    bytes are 2^64 - 2^40 bytes. Such an arena is refused, with or without backing."""
    lib = _native.load()
    handle = ctypes.c_void_p()
    _native.set_option("rank_stride_align", 1 << 40)
    try:
        stride = 986_895 << 40
        assert 17 * stride == (1 << 64) - (1 << 40)
        for flags in (_native.ODC_ARENA_DRY_RUN, _native.ODC_ARENA_NO_BACKING):
            assert lib.odc_arena_create(17, stride, flags, ctypes.byref(handle)) == _native.ODC_ERR_INVALID
            assert "overflows" in lib.odc_last_error().decode() and not handle.value
        # one region fewer fits
        _native.check(lib.odc_arena_create(16, stride, _native.ODC_ARENA_NO_BACKING, ctypes.byref(handle)))
        _native.check(lib.odc_arena_destroy(handle))
    finally:
        _native.set_option("rank_stride_align", 16384)


@pytest.mark.parametrize("n_items", [5, 256, 257, 700])
def test_accumulate_item_lists_with_tiny_items_keep_every_item(arena, n_items):
    """Items of less than one tile per rank are launched after the others (also through the
    heap-allocated order of lists longer than 256): launches and tiles still add up, and an item
    that is too large is still reported under the caller's index."""
    W = 4
    a = arena(W, 1 << 46)
    sizes = [(100 if i % 3 == 0 else 0 if i % 7 == 0 else 5000 + i) for i in range(n_items)]
    items = (_native.AccumItem * n_items)()
    off = 0
    for it, sz in zip(items, sizes):
        it.grad, it.grad_elems, it.acc_offset, it.shard_elems = OUTSIDE, W * sz, off, sz
        off += -(-4 * sz // 256) * 256
    _native.check(a.lib.odc_scatter_accumulate(a.handle, items, n_items, _native.DTYPE_BF16, _native.DTYPE_F32, None))
    nonempty = [s for s in sizes if s]
    launches, tiles, _ = a.counters()
    assert launches == math.ceil(len(nonempty) / _native.MAX_ITEMS_PER_LAUNCH)
    assert tiles == W * sum(math.ceil(s / TILE_ELEMS) for s in nonempty)
    bad = n_items - 2  # position in the caller's list; in launch order it sits elsewhere
    items[bad].shard_elems = (1 << 31) * TILE_ELEMS // W  # 2^31 tiles in all: one too many for a launch
    items[bad].grad_elems, items[bad].acc_offset = 0, 0
    status = a.lib.odc_scatter_accumulate(a.handle, items, n_items, _native.DTYPE_BF16, _native.DTYPE_F32, None)
    message = a.lib.odc_last_error().decode()
    assert status == _native.ODC_ERR_INVALID and f"item {bad}:" in message and "too large for one launch" in message
