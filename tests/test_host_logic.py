"""Host-side logic that needs no GPU: the C ABI surface, the arena's offset bookkeeping (on an
arena without device memory), the registry and splitter mirrors, error behaviour, and the rule
that the product never reaches for the oracle or a CPU fallback."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

from odc_amd import _native
from odc_amd.primitives import utils
from oracle import odc_oracle as oracle

ROOT = Path(__file__).resolve().parent.parent


# ---- C ABI -------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "odc_hip.h").read_text()
    declared = set(re.findall(r"\b(odc_[a-z_]+)\s*\(", header))
    assert declared == set(_native.EXPORTED_SYMBOLS)
    lib = _native.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/odc_hip.h but not exported"
    assert lib.odc_abi_version() == _native.ABI_VERSION == int(re.search(r"ODC_HIP_ABI_VERSION (\d+)", header).group(1))
    assert _native.MAX_ITEMS_PER_LAUNCH == int(re.search(r"ODC_MAX_ITEMS_PER_LAUNCH (\d+)", header).group(1))


def test_header_is_plain_c():
    import subprocess

    subprocess.run(
        ["gcc", "-std=c99", "-fsyntax-only", "-Wall", "-Wextra", "-pedantic", "-x", "c",
         str(ROOT / "include" / "odc_hip.h")],
        check=True,
    )


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(_native.GatherItem) == 24
    assert ctypes.sizeof(_native.AccumItem) == 32
    assert ctypes.sizeof(_native.Span) == 16
    assert ctypes.sizeof(_native.ArenaInfo) == 4 * 4 + 5 * 8


def test_options_roundtrip_and_unknown_name():
    old = _native.get_option("gather_blocks_per_cu")
    _native.set_option("gather_blocks_per_cu", 3)
    assert _native.get_option("gather_blocks_per_cu") == 3
    _native.set_option("gather_blocks_per_cu", old)
    with pytest.raises(_native.OdcNativeError) as e:
        _native.set_option("no_such_knob", 1)
    assert e.value.code == _native.ODC_ERR_INVALID and "no_such_knob" in e.value.message
    with pytest.raises(_native.OdcNativeError):
        _native.set_option("rank_major", -1)
    for name in ("rank_stagger_bytes", "rank_stride_align", "alloc_align"):
        with pytest.raises(_native.OdcNativeError):  # would wrap the arena's address arithmetic
            _native.set_option(name, (1 << 62) + 1)


# ---- arena bookkeeping (no device memory) ------------------------------------------------------
def test_arena_offsets_first_fit_and_coalescing():
    a = utils.SymmetricArena(8, 1 << 20, backing=False)
    info = a.info()
    assert (info.world_size, info.device, info.base, info.bytes_per_rank) == (8, -1, 0, 1 << 20)
    assert info.rank_stride >= info.bytes_per_rank
    o = [a.alloc(n) for n in (100, 1000, 1, 0, 4096)]
    assert o == [0, 256, 1280, 1536, 1792]  # 256 B granules, bump order
    assert a.info().bytes_in_use == 256 + 1024 + 256 + 256 + 4096 and a.info().n_allocations == 5
    a.free(o[1])
    a.free(o[2])  # merges with the freed block before it
    assert a.alloc(1280) == 256  # fits exactly into the merged hole
    a.free(o[0])
    assert a.alloc(10) == 0
    with pytest.raises(_native.OdcNativeError) as e:
        a.free(12345)
    assert e.value.code == _native.ODC_ERR_NOT_FOUND
    hw = a.info().high_water
    a.reset()
    assert a.info().bytes_in_use == 0 and a.info().n_allocations == 0 and a.info().high_water == hw
    assert a.alloc(1 << 20) == 0
    with pytest.raises(_native.OdcNativeError) as e:
        a.alloc(1)
    assert e.value.code == _native.ODC_ERR_NOMEM
    a.destroy()
    with pytest.raises(RuntimeError):
        a.alloc(1)  # use after finalize


@pytest.mark.parametrize("big_align", [256, 4096, 16384, 65536])
@pytest.mark.parametrize("seed", range(4))
def test_arena_random_schedule_against_a_model(seed, big_align):
    """Random allocs and frees checked against a plain first-fit model (256 B granules; buffers of
    `alloc_align` bytes or more, by default a tile, start on multiples of it): same offsets, no live ranges overlapping, in-use
    and high-water figures, full coalescing at the end."""
    import random

    rng = random.Random(seed)
    cap = 1 << 20
    _native.set_option("alloc_align", big_align)  # read when the arena is created
    try:
        a = utils.SymmetricArena(3, cap, backing=False)
    finally:
        _native.set_option("alloc_align", 16384)
    live = {}  # offset -> rounded size
    high = 0

    def model_alloc(n):
        need = max(256, (n + 255) // 256 * 256)
        align = big_align if need >= big_align else 256
        cursor = 0
        for off in sorted(live) + [cap]:  # the free blocks are the gaps between live ranges
            start = (cursor + align - 1) // align * align
            if off > cursor and start + need <= off:
                return start, need
            cursor = off + live.get(off, 0)
        return None, need

    for _ in range(600):
        if live and rng.random() < 0.45:
            off = rng.choice(sorted(live))
            a.free(off)
            del live[off]
        else:
            n = rng.choice([0, 1, 255, 256, 257, 4096, 10_000, 70_000, 200_000])
            want, need = model_alloc(n)
            if want is None:
                with pytest.raises(_native.OdcNativeError) as e:
                    a.alloc(n)
                assert e.value.code == _native.ODC_ERR_NOMEM
            else:
                assert a.alloc(n) == want
                live[want] = need
                high = max(high, want + need)
        info = a.info()
        assert info.n_allocations == len(live) and info.bytes_in_use == sum(live.values())
        assert info.high_water == high
    for off in list(live):
        a.free(off)
    assert a.alloc(cap) == 0  # everything merged back into one block
    a.destroy()


def test_arena_places_large_buffers_on_tile_boundaries():
    a = utils.SymmetricArena(4, 1 << 20, backing=False)
    assert a.info().rank_stride % 16384 == 0
    assert a.alloc(100) == 0
    assert a.alloc(16384) == 16384  # skips to the next tile boundary
    assert a.alloc(300) == 256  # the gap in front is still usable
    assert a.alloc(16383) == 32768  # rounds to 16384 bytes: aligned like the others, so not in the gap
    assert a.alloc(15616) == 768  # under a tile: 256 B granules, fills the gap exactly
    a.destroy()
    _native.set_option("alloc_align", 256)
    _native.set_option("rank_stride_align", 256)
    try:
        b = utils.SymmetricArena(4, 1 << 20, backing=False)
        assert [b.alloc(n) for n in (100, 16384, 300)] == [0, 256, 16640]
        b.destroy()
    finally:
        _native.set_option("alloc_align", 16384)
        _native.set_option("rank_stride_align", 16384)


def test_arena_is_safe_to_share_between_host_threads():
    """The primitives are called from the main thread and from autograd's device thread
    (FSDP post-backward hooks): concurrent alloc/free/locate-style bookkeeping must keep the
    allocator consistent. ctypes releases the GIL during the calls."""
    import random
    import threading

    a = utils.SymmetricArena(2, 64 << 20, backing=False)
    errors, held = [], [[] for _ in range(8)]

    def worker(t):
        rng = random.Random(t)
        try:
            for _ in range(2000):
                if held[t] and rng.random() < 0.5:
                    a.free(held[t].pop(rng.randrange(len(held[t]))))
                else:
                    n = rng.choice([1, 300, 5000, 40_000])
                    held[t].append((a.alloc(n), n)[0])
                a.info()
        except Exception as e:  # noqa: BLE001 - reported below, on the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    offsets = [o for h in held for o in h]
    assert len(offsets) == len(set(offsets)) == a.info().n_allocations  # nothing handed out twice
    for o in offsets:
        a.free(o)
    assert a.info().bytes_in_use == 0 and a.alloc(64 << 20) == 0
    a.destroy()


def test_sizing_run_for_the_8b_layer():
    """What the bookkeeping-only arena is for: learn the bytes per rank a workload needs."""
    from odc_amd.workloads import llama3_8b_layer_shapes, numel

    W = 8
    a = utils.SymmetricArena(W, 1 << 40, backing=False)
    for _, shape in llama3_8b_layer_shapes():
        a.alloc(numel(shape) // W * 2)  # bf16 shard
        a.alloc(numel(shape) // W * 4)  # fp32 accumulation
    need = a.info().high_water
    assert 27_264_000 * 6 <= need <= 27_264_000 * 6 + 18 * 16384  # tile-sized buffers start on 16 KiB boundaries
    a.destroy()


def test_bad_arguments_and_compute_on_unbacked_arena():
    lib = _native.load()
    h = ctypes.c_void_p()
    assert lib.odc_arena_create(0, 1024, 0, ctypes.byref(h)) == _native.ODC_ERR_INVALID
    assert lib.odc_arena_create(4, 0, 0, ctypes.byref(h)) == _native.ODC_ERR_INVALID
    for absurd in ((1 << 64) - 1, (1 << 63), (1 << 60) + 1):  # sizes whose rounding or product would wrap
        assert lib.odc_arena_create(4, absurd, _native.ODC_ARENA_NO_BACKING, ctypes.byref(h)) == _native.ODC_ERR_INVALID
    assert lib.odc_arena_create(4, 1024, 0x80, ctypes.byref(h)) == _native.ODC_ERR_INVALID
    assert lib.odc_arena_create(4, 1024, 0, None) == _native.ODC_ERR_INVALID
    assert lib.odc_arena_destroy(None) == _native.ODC_ERR_INVALID
    a = utils.SymmetricArena(4, 1 << 16, backing=False)
    items = (_native.GatherItem * 1)()
    assert lib.odc_gather(a.handle, items, 1, 0, None) == _native.ODC_ERR_NO_BACKING
    acc = (_native.AccumItem * 1)()
    assert lib.odc_scatter_accumulate(a.handle, acc, 1, 0, 2, None) == _native.ODC_ERR_NO_BACKING
    spans = (_native.Span * 1)()
    assert lib.odc_clear(a.handle, spans, 1, None) == _native.ODC_ERR_NO_BACKING
    assert b"no device memory" in lib.odc_last_error()
    assert lib.odc_arena_ptr(a.handle, 0, 0) is None
    assert lib.odc_arena_locate(a.handle, ctypes.c_void_p(64), None, None, None) == _native.ODC_ERR_NO_BACKING
    with pytest.raises(RuntimeError):
        a.view(0, 0, (4,), torch.float32)
    a.destroy()


def test_product_fails_loudly_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("this check is for the CPU-only container")
    with pytest.raises(RuntimeError):
        utils.init_nvshmem(world_size=4, symmetric_size="1M")
    with pytest.raises(_native.OdcNativeError) as e:
        utils.SymmetricArena(4, 1 << 20)  # hipMalloc has no device to run on
    assert e.value.code == _native.ODC_ERR_HIP
    with pytest.raises(RuntimeError):
        utils.get_rank()  # no world


def test_product_never_imports_the_oracle():
    for path in (ROOT / "odc_amd").rglob("*"):
        if path.suffix in (".py", ".hip", ".h", ".cpp"):
            text = path.read_text()
            assert "oracle" not in text.lower(), f"{path} mentions the oracle"
    assert "oracle" not in (ROOT / "include" / "odc_hip.h").read_text().lower()


# ---- mirrors of the reference's host classes ---------------------------------------------------
@pytest.mark.parametrize("env,shape,W", [
    (None, (27_264_000,), 8), (None, (7_340_032,), 8), (None, (512,), 8), (None, (100,), 8),
    ("0", (100,), 8), ("-1", (1000, 3), 12), ("1024", (1000, 3), 4), (None, (218_112_000,), 8),
    ("4096", (10,), 64),
])
def test_buffer_splitter_matches_the_oracle(monkeypatch, env, shape, W):
    if env is None:
        monkeypatch.delenv("ODC_MAX_BUFFER_SIZE", raising=False)
    else:
        monkeypatch.setenv("ODC_MAX_BUFFER_SIZE", env)
    mine, ref = utils.BufferSplitter(), oracle.BufferSplitter()
    assert mine.get_global_buffer_size(shape) == ref.get_global_buffer_size(shape)
    assert mine.get_local_buffer_size(shape, W) == ref.get_local_buffer_size(shape, W)


def test_buffer_splitter_assertion(monkeypatch):
    monkeypatch.delenv("ODC_MAX_BUFFER_SIZE", raising=False)
    with pytest.raises(AssertionError, match="ODC_MAX_BUFFER_SIZE"):
        utils.BufferSplitter().get_local_buffer_size((100,), 12)


def test_parse_size():
    assert utils.parse_size("30G") == 30 * 2**30
    assert utils.parse_size("5000000000") == 5_000_000_000
    assert utils.parse_size("512m") == 512 * 2**20
    assert utils.parse_size("1.5GB") == int(1.5 * 2**30)
    assert utils.parse_size(4096) == 4096


class _HostArena:
    """Stand-in arena over host memory, for the registry's bookkeeping only."""

    def __init__(self, world_size, nbytes):
        self.world_size = world_size
        self.mem = [torch.zeros(nbytes, dtype=torch.uint8) for _ in range(world_size)]
        self.top = 0
        self.freed = []

    def alloc(self, nbytes):
        off = self.top
        self.top += max(256, -(-nbytes // 256) * 256)
        return off

    def free(self, offset):
        self.freed.append(offset)

    def view(self, rank, offset, shape, dtype):
        n = torch.Size(shape).numel() * dtype.itemsize
        return self.mem[rank][offset : offset + n].view(dtype).view(shape)


def test_registry_bookkeeping_on_a_host_arena():
    current = {"rank": 0}
    reg = utils.SymmBufferRegistry(arena=_HostArena(3, 1 << 16), rank_fn=lambda: current["rank"])
    t = reg.allocate_symm_buffer("w", (10,), torch.float32)
    assert reg.has_key("w") and not reg.has_key("x") and reg.is_nvshmem_tensor(t)
    with pytest.raises(AssertionError):
        reg.allocate_symm_buffer("w", (10,), torch.float32)  # utils.py:127
    with pytest.raises(ValueError, match="not found"):
        reg.get_symm_buffer("x")  # utils.py:153-156
    assert reg.get_or_create_symm_buffer("w", (10,), torch.float32).data_ptr() == t.data_ptr()
    peers = reg.get_peer_tensors(t)
    assert len(peers) == 3 and len({p.data_ptr() for p in peers}) == 3
    # update copies once per rank until flush (utils.py:103-116)
    assert torch.equal(reg.update_symm_buffer("w", torch.arange(10.0)), torch.arange(10.0))
    assert torch.equal(reg.update_symm_buffer("w", torch.zeros(10)), torch.arange(10.0))
    current["rank"] = 2
    assert torch.equal(reg.update_symm_buffer("w", torch.ones(10)), torch.ones(10))  # rank 2's first
    assert torch.equal(peers[0], torch.arange(10.0)) and not peers[1].any()
    assert reg.get_symm_buffer("w").data_ptr() == peers[2].data_ptr()
    assert reg.local_tensor["w"].data_ptr() == peers[2].data_ptr()
    reg.flush()
    assert torch.equal(reg.update_symm_buffer("w", torch.full((10,), 7.0)), torch.full((10,), 7.0))
    reg.update_symm_buffer(("k", 1), torch.zeros(4, dtype=torch.bfloat16))  # lazily allocates
    assert reg.memory_allocated() == 40 + 8
    reg.finalize()
    assert sorted(reg._arena.freed) == [0, 256] and not reg.has_key("w") and reg.memory_allocated() == 0


def test_services_refuse_host_tensors():
    from odc_amd import GatherService, ReductionService

    if utils.is_initialized():
        pytest.skip("a world exists")
    with pytest.raises(RuntimeError):  # no arena, no compute
        GatherService().gather_into_tensor(torch.empty(8), torch.empty(2), utils.VirtualGroup(4))
    with pytest.raises(RuntimeError):
        ReductionService().scatter_accumulate("k", torch.empty(8), utils.VirtualGroup(4))


def test_workload_shapes():
    from odc_amd import workloads as w

    assert sum(w.numel(s) for _, s in w.llama3_8b_layer_shapes()) == 218_112_000
    assert sum(w.numel(s) for _, unit in w.llama3_8b_units() for _, s in unit) == 8_030_261_248
    sizes = w.uneven_flat_numels()
    assert len(sizes) == 40 and all(4096 <= n <= 58_720_256 + 12 and n % 12 for n in sizes)
    assert sizes == w.uneven_flat_numels()  # deterministic


def test_small_helpers(monkeypatch):
    """Closed forms and environment lookups that nothing else touches: the splitter's rounding
    (utils.py:229-230), the node-size lookup (utils.py:195-199) and the symmetric-tensor tag
    (utils.py:118-124)."""
    s = utils.BufferSplitter()
    assert [s.round_to_data_size(n) for n in (0, 1, 63, 64, 65, 100, 128)] == [0, 64, 64, 64, 128, 128, 128]
    if not utils.is_initialized():
        monkeypatch.delenv("RAY_LOCAL_WORLD_SIZE", raising=False)
        monkeypatch.setenv("LOCAL_WORLD_SIZE", "8")
        assert utils.get_local_world_size() == 8
        monkeypatch.setenv("RAY_LOCAL_WORLD_SIZE", "4")  # Ray's variable wins, as in the reference
        assert utils.get_local_world_size() == 4
        with pytest.raises(RuntimeError):
            utils.get_world_size()
    t = torch.zeros(3)
    assert not utils.SymmBufferRegistry.is_nvshmem_tensor(t)
    utils.SymmBufferRegistry.set_nvshmem_flag(t)
    assert utils.SymmBufferRegistry.is_nvshmem_tensor(t)
    monkeypatch.setenv("ODC_COMM_STREAM", "nonsense")
    with pytest.raises(ValueError):
        utils.launch_stream_policy()
    monkeypatch.setenv("ODC_COMM_STREAM", "dedicated")
    assert utils.launch_stream_policy() == "dedicated"
    monkeypatch.delenv("ODC_COMM_STREAM")
    assert utils.launch_stream_policy() == "caller"


def test_fsdp2_accumulation_slices_start_on_tiles():
    """The FSDP2 group accumulation: slices of a tile (4096 elements) or more start on a multiple
    of the tile, smaller ones are packed."""
    from odc_amd.fsdp.fsdp2 import tile_aligned_offsets

    assert tile_aligned_offsets([512, 4096, 10, 5000, 4095, 8192]) == ([0, 4096, 8192, 12288, 17288, 24576], 32768)
    assert tile_aligned_offsets([3, 5, 7]) == ([0, 3, 8], 15)
    assert tile_aligned_offsets([]) == ([], 0)
    assert tile_aligned_offsets([4096, 4096]) == ([0, 4096], 8192)


def test_under_the_sanitizer_run_the_sanitized_library_is_the_one_loaded():
    """tests/test_host_sanitizers.py runs this file against a g++ AddressSanitizer + UBSan build of
    the host side; there, prove that this build (and the sanitizer runtime) is what is mapped."""
    import os

    if os.environ.get("ODC_EXPECT_SANITIZED") != "1":
        pytest.skip("only meaningful inside the sanitizer run")
    _native.load()
    maps = open("/proc/self/maps").read()
    assert os.environ["ODC_HIP_LIBRARY"] in maps and "libasan" in maps
    assert str(_native.CSRC_DIR / "libodc_hip.so") not in maps


def test_the_reference_module_paths_resolve_to_this_package():
    """``odc`` is an alias package without logic: the module paths the reference's callers import
    (examples/all_gather.py:10-11, examples/reduce_scatter.py:9-10, examples/FSDP2/example.py:15-17)
    are the odc_amd modules themselves."""
    import importlib

    import odc
    import odc_amd

    for name in ("primitives", "primitives.gather", "primitives.scatter_accumulate", "primitives.utils",
                 "primitives.tensor_ipc", "fsdp", "fsdp.fsdp1", "fsdp.fsdp2"):
        assert importlib.import_module(f"odc.{name}") is importlib.import_module(f"odc_amd.{name}"), name
    from odc.fsdp import fsdp2
    from odc.primitives.gather import GatherService
    from odc.primitives.utils import SymmBufferRegistry, init_nvshmem

    assert GatherService is odc_amd.GatherService and SymmBufferRegistry is odc_amd.SymmBufferRegistry
    assert init_nvshmem is odc_amd.init_nvshmem is odc.init_nvshmem and fsdp2.patch_fsdp2
    text = (ROOT / "odc" / "__init__.py").read_text()
    assert "def " not in text and "class " not in text, "the alias package holds no logic"


def test_stream_order_waits_only_when_a_key_changes_streams(monkeypatch):
    """``StreamOrder`` (the per-key memory of the last writing stream) on the CPU, with the two
    functions that touch the GPU replaced: launches that stay on one stream join nothing; a key
    that moves to another stream joins exactly the stream it was last written on, once; a launch
    over all keys collapses the table; keys never seen count as written on the first stream."""
    joins = []
    monkeypatch.setattr(utils, "stream_from_handle", lambda handle: ("stream", handle))
    monkeypatch.setattr(utils, "join_streams", lambda current, previous: joins.append((current[1], previous)))
    order = utils.StreamOrder()
    A, B, C = 0x10, 0x20, 0x30
    for _ in range(3):
        order.before_launch(["a", "b"], A, total=3)
    assert joins == [] and not order._last
    order.before_launch(["a"], B, total=3)          # a: A -> B
    assert joins == [(B, A)]
    order.before_launch(["a"], B, total=3)          # stays: nothing
    order.before_launch(["b"], A, total=3)          # b never left A
    assert joins == [(B, A)]
    order.before_launch(["a", "b"], C, total=3)     # a from B, b from A: two joins, in any order
    assert sorted(joins[1:]) == [(C, A), (C, B)]
    joins.clear()
    order.before_launch(["c"], C, total=3)          # c counts as written on the first stream, A
    assert joins == [(C, A)]
    assert not order._last and order._base == C, "all three keys on C: the table collapses"
    joins.clear()
    order.before_launch(["a"], A, total=3)
    order.before_launch(["a", "b", "c"], B, all_keys=True, total=3)   # e.g. a clear of everything
    assert sorted(joins) == [(A, C), (B, A), (B, C)]
    assert not order._last and order._base == B
    joins.clear()
    order.before_launch(["b"], B, total=3)
    assert joins == []
    order.forget()
    order.before_launch(["a"], C, total=3)
    assert joins == [] and order._base == C
