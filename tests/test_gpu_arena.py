"""The symmetric arena and registry on the GPU, through the C ABI."""


import pytest
import torch

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu


def test_symmetric_offsets_and_views(make_world):
    from odc_amd import SymmBufferRegistry, virtual_rank
    from odc_amd.primitives import utils

    W = 5
    make_world(W, 1 << 20)
    arena = utils.get_world().arena
    reg = SymmBufferRegistry.get_instance()
    a = reg.allocate_symm_buffer("a", (1000,), torch.float32)
    b = reg.allocate_symm_buffer("b", (3, 5), torch.bfloat16)
    assert reg.is_nvshmem_tensor(a) and a.shape == (1000,) and b.shape == (3, 5)
    peers = reg.get_peer_tensors(a)
    assert len(peers) == W and peers[0].data_ptr() == a.data_ptr()
    stride = arena.info().rank_stride
    for r, t in enumerate(peers):
        assert t.data_ptr() == arena.ptr(r, reg.get_offset("a")) == a.data_ptr() + r * stride
        assert arena.locate(t.data_ptr() + 40) == (r, reg.get_offset("a"), 40)
    with virtual_rank(3):
        assert reg.get_symm_buffer("a").data_ptr() == peers[3].data_ptr()
        assert reg.get_peer_tensors(reg.get_symm_buffer("a")) is peers
    # writes through one rank's view land only in that rank's region
    for r, t in enumerate(peers):
        t.fill_(float(r))
    for r, t in enumerate(peers):
        assert (t.cpu() == r).all()
    with pytest.raises(AssertionError):
        reg.allocate_symm_buffer("a", (1,), torch.float32)  # utils.py:127
    with pytest.raises(ValueError):
        reg.get_symm_buffer("missing")  # utils.py:153-156
    assert reg.memory_allocated() == 1000 * 4 + 15 * 2


def test_update_symm_buffer_copies_once_until_flush(make_world):
    """utils.py:103-116."""
    from odc_amd import SymmBufferRegistry

    make_world(2, 1 << 20)
    reg = SymmBufferRegistry.get_instance()
    t = reg.update_symm_buffer(7, torch.arange(10.0).cuda())
    assert_bit_equal(t, torch.arange(10.0), "first update copies")
    t2 = reg.update_symm_buffer(7, torch.zeros(10).cuda())
    assert t2.data_ptr() == t.data_ptr()
    assert_bit_equal(t2, torch.arange(10.0), "second update is a no-op")
    reg.flush()
    assert_bit_equal(reg.update_symm_buffer(7, torch.ones(10).cuda()), torch.ones(10), "after flush")


def test_arena_exhaustion_and_bad_arguments(make_world):
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry, _native
    from odc_amd.primitives import utils

    group = make_world(4, 1 << 16)
    reg = SymmBufferRegistry.get_instance()
    with pytest.raises(_native.OdcNativeError) as e:
        reg.allocate_symm_buffer("big", (1 << 20,), torch.float32)
    assert e.value.code == _native.ODC_ERR_NOMEM and "ODC_SYMMETRIC_SIZE" in str(e.value)
    src = reg.allocate_symm_buffer("s", (64,), torch.bfloat16)
    gather = GatherService()
    with pytest.raises(AssertionError):  # output numel must be W * shard numel
        gather.gather_into_tensor(torch.empty(100, dtype=torch.bfloat16, device="cuda"), src, group)
    with pytest.raises(ValueError):  # input must live in the arena
        gather.gather_into_tensor(torch.empty(256, dtype=torch.bfloat16, device="cuda"),
                                  torch.empty(64, dtype=torch.bfloat16, device="cuda"), group)
    red = ReductionService(accumulation_dtype=torch.float32)
    with pytest.raises(AssertionError):  # shape[0] % W (scatter_accumulate.py:589-592)
        red.scatter_accumulate("k", torch.zeros(10, dtype=torch.bfloat16, device="cuda"), group)
    with pytest.raises(TypeError):
        red.scatter_accumulate("k", torch.zeros(8, dtype=torch.int32, device="cuda"), group)
    # raw C ABI: offsets outside the rank region are refused, nothing is launched
    lib = _native.load()
    arena = utils.get_world().arena
    item = (_native.GatherItem * 1)()
    item[0].dst = src.data_ptr()
    item[0].src_offset = 1 << 16
    item[0].shard_bytes = 64
    assert lib.odc_gather(arena.handle, item, 1, 0, None) == _native.ODC_ERR_INVALID
    assert lib.odc_gather(arena.handle, item, 1, 9, None) == _native.ODC_ERR_INVALID  # first_rank >= W
    # dst overlapping a shard it reads
    item[0].src_offset = reg.get_offset("s")
    item[0].shard_bytes = 32
    assert lib.odc_gather(arena.handle, item, 1, 0, None) == _native.ODC_ERR_INVALID
    assert b"overlaps" in lib.odc_last_error()
    # element counts whose byte size wraps around 2**64 are refused like any other overrun
    grad = torch.zeros(256, dtype=torch.bfloat16, device="cuda")
    for elems in (1 << 62, (1 << 63) + 16, (1 << 64) - 1):
        acc = (_native.AccumItem * 1)()
        acc[0].grad, acc[0].grad_elems, acc[0].acc_offset, acc[0].shard_elems = grad.data_ptr(), 256, 0, elems
        assert lib.odc_scatter_accumulate(arena.handle, acc, 1, _native.DTYPE_BF16, _native.DTYPE_F32, None) \
            == _native.ODC_ERR_INVALID
        assert b"exceed" in lib.odc_last_error()
        cast = (_native.GatherCastItem * 1)()
        cast[0].dst, cast[0].src_offset, cast[0].shard_elems = grad.data_ptr(), 0, elems
        assert lib.odc_gather_cast(arena.handle, cast, 1, _native.DTYPE_F32, _native.DTYPE_BF16, 0, None) \
            == _native.ODC_ERR_INVALID
        pub = (_native.PublishItem * 1)()
        pub[0].acc_offset, pub[0].elems, pub[0].out = 0, elems, None
        assert lib.odc_publish(arena.handle, 0, pub, 1, _native.DTYPE_F32, _native.DTYPE_F32, 2.0, None) \
            == _native.ODC_ERR_INVALID
    torch.cuda.synchronize()


def test_gather_from_inner_view_and_multi_item(make_world):
    """A shard that is a slice of a larger symmetric buffer resolves through odc_arena_locate."""
    from odc_amd import GatherService, SymmBufferRegistry, virtual_rank

    W = 3
    group = make_world(W, 1 << 20)
    reg = SymmBufferRegistry.get_instance()
    reg.allocate_symm_buffer("g", (1000,), torch.int32)
    for r in range(W):
        with virtual_rank(r):
            reg.get_symm_buffer("g").copy_(torch.arange(1000, dtype=torch.int32) + 10_000 * r)
    local = reg.get_symm_buffer("g")
    out_a = torch.empty(W * 100, dtype=torch.int32, device="cuda")
    out_b = torch.empty(W * 7, dtype=torch.int32, device="cuda")
    GatherService().gather_into_tensors([out_a, out_b], [local[50:150], local[993:1000]], group)
    for r in range(W):
        assert_bit_equal(out_a[r * 100 : (r + 1) * 100], torch.arange(50, 150, dtype=torch.int32) + 10_000 * r)
        assert_bit_equal(out_b[r * 7 : (r + 1) * 7], torch.arange(993, 1000, dtype=torch.int32) + 10_000 * r)


def test_plain_c_client_of_the_abi():
    """tests/c_abi/abi_check.c, built with gcc by build(): the library without Python or torch."""
    import subprocess
    from pathlib import Path

    exe = Path(__file__).resolve().parent / "c_abi" / "abi_check"
    if not exe.exists():  # nothing built yet
        import __graft_entry__

        __graft_entry__.build_c_client()
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "abi_check ok" in proc.stdout


def test_reference_named_symmetric_tensor_helpers(make_world):
    """nvshmem_create_tensor / get_same_node_tensors / nvshmem_free_tensor_sync / get_local_world_pg
    (odc/primitives/utils.py:53-81,178-192) on the arena: peers alias one offset in W regions."""
    import torch

    from odc_amd import virtual_rank
    from odc_amd.primitives import utils

    W = 4
    group = make_world(W, 1 << 20)
    with virtual_rank(2):
        mine = utils.nvshmem_create_tensor((3, 5), torch.float32)
        peers = utils.get_same_node_tensors(mine, 2, W)
    assert len(peers) == W and peers[2] is mine
    arena = utils.get_world().arena
    offsets = set()
    for r, t in enumerate(peers):
        t.fill_(float(r))
        rank, off, inner = arena.locate(t.data_ptr())
        assert rank == r and inner == 0 and tuple(t.shape) == (3, 5)
        offsets.add(off)
    assert len(offsets) == 1  # symmetric: the same offset in every rank region
    for r, t in enumerate(peers):
        assert (t == float(r)).all()
    # a registry buffer works as the handle too, from any rank's view
    reg = utils.SymmBufferRegistry.get_instance()
    buf = reg.allocate_symm_buffer("x", (8,), torch.int32)
    views = utils.get_same_node_tensors(buf, utils.get_rank(), W)
    for r, (a, b) in enumerate(zip(views, reg.peer_tensors["x"])):
        assert a.data_ptr() == b.data_ptr(), r
    assert utils.get_local_world_pg(group) is group
    before = arena.info().n_allocations
    utils.nvshmem_free_tensor_sync(mine)
    assert arena.info().n_allocations == before - 1
    with pytest.raises(ValueError):
        utils.nvshmem_free_tensor_sync(mine)


def test_tensor_ipc_handles_round_trip(make_world):
    """get_ipc_handle / reconstruct_tensor (csrc/tensor_ipc/tensor_ipc.cu:24-57) inside one
    process: 72-byte handles of whole buffers and of inner views, for every rank."""
    import torch

    from odc_amd import SymmBufferRegistry, virtual_rank
    from odc_amd.primitives import get_ipc_handle, reconstruct_tensor

    W = 3
    make_world(W, 1 << 20)
    reg = SymmBufferRegistry.get_instance()
    reg.allocate_symm_buffer("acc", (1000,), torch.float32)
    for r, peer in enumerate(reg.peer_tensors["acc"]):
        peer.copy_(torch.arange(1000, dtype=torch.float32) + 1000 * r)
    for r in range(W):
        with virtual_rank(r):
            local = reg.get_symm_buffer("acc")
        handle = get_ipc_handle(local)
        assert isinstance(handle, bytes) and len(handle) == 72
        again = reconstruct_tensor(handle, (1000,), torch.float32)
        assert again.data_ptr() == local.data_ptr() and torch.equal(again, local)
        inner = get_ipc_handle(local[100:])  # the reference adds the pointer's offset to the handle
        part = reconstruct_tensor(inner, (10, 5), torch.float32)
        assert torch.equal(part.reshape(-1), local[100:150])
        as_bytes = reconstruct_tensor(inner, (8,), torch.uint8)
        assert torch.equal(as_bytes, local[100:102].view(torch.uint8))
    with pytest.raises(ValueError):
        reconstruct_tensor(b"\0" * 72, (1,), torch.float32)
    with pytest.raises(ValueError):
        reconstruct_tensor(handle[:10], (1,), torch.float32)
    with pytest.raises(Exception):
        get_ipc_handle(torch.zeros(4, device="cuda"))  # not in the arena


def test_regions_and_large_buffers_start_on_tile_boundaries(make_world):
    """Rank regions and every buffer of a tile (16 KiB) or more start on a multiple of 16 KiB of
    the device address space, whatever alignment hipMalloc returned."""
    from odc_amd import SymmBufferRegistry
    from odc_amd.primitives import utils

    make_world(5, 3 << 20)
    arena = utils.get_world().arena
    assert arena.base % 16384 == 0 and arena.rank_stride % 16384 == 0
    registry = SymmBufferRegistry.get_instance()
    registry.allocate_symm_buffer("small", (100,), torch.float32)
    registry.allocate_symm_buffer("big", (5000,), torch.float32)
    registry.allocate_symm_buffer("small2", (3,), torch.bfloat16)
    registry.allocate_symm_buffer("big2", (8192,), torch.bfloat16)
    for key in ("big", "big2"):
        for peer in registry.peer_tensors[key]:
            assert peer.data_ptr() % 16384 == 0
    for key in ("small", "small2"):
        for peer in registry.peer_tensors[key]:
            assert peer.data_ptr() % 256 == 0


def test_a_service_kept_across_arenas_does_not_reuse_stale_plans(make_world):
    """Launch plans and shard offsets are cached inside the services; an arena created after
    finalize_distributed() may hand out the same addresses for other offsets and another W."""
    from helpers import assert_bit_equal, put_shards
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry
    from odc_amd.primitives import utils
    from oracle import odc_oracle as oracle

    gather, reduction = GatherService(), ReductionService(accumulation_dtype=torch.float32)
    g = torch.Generator().manual_seed(9)
    S = 20_000
    for W, pad in ((4, 0), (2, 4096), (4, 0)):
        group = make_world(W, 4 << 20)
        registry = SymmBufferRegistry.get_instance()
        if pad:
            registry.allocate_symm_buffer("pad", (pad,), torch.uint8)  # shifts every later offset
        shards = [torch.randn(S, generator=g).bfloat16() for _ in range(W)]
        src = put_shards(registry, "p", shards)
        out = torch.empty(W * S, dtype=torch.bfloat16, device="cuda")
        gather.gather_into_tensor(out, src, group)
        assert_bit_equal(out, oracle.gather(shards), f"gather at W={W}")
        fresh = ReductionService(accumulation_dtype=torch.float32)  # accumulations belong to one arena
        grad = torch.randn(W * S, generator=g).bfloat16()
        fresh.scatter_accumulate("k", grad.cuda(), group)
        want = [torch.zeros(S) for _ in range(W)]
        oracle.scatter_accumulate(want, grad)
        for r, acc in enumerate(fresh.get_peer_accumulations("k")):
            assert_bit_equal(acc, want[r], f"accumulation of rank {r} at W={W}")
        torch.cuda.synchronize()
        registry.finalize()
        utils.finalize_distributed()
    del reduction


def test_importing_the_package_before_torch_still_finds_the_gpu():
    """A fresh interpreter that imports odc_amd (which loads libodc_hip.so) BEFORE torch must end
    up with ONE HIP runtime, torch's: the arena is created and torch sees the same device."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    code = "\n".join([
        f"import sys; sys.path.insert(0, {str(root)!r})",
        "assert 'torch' not in sys.modules",
        "import odc",
        "import torch",
        "g = odc.init_nvshmem(world_size=2, symmetric_size=1 << 20)",
        "t = odc.SymmBufferRegistry.get_instance().allocate_symm_buffer('k', (16,), torch.float32)",
        "t.fill_(3.0); torch.cuda.synchronize(); assert float(t.sum()) == 48.0",
        "odc.SymmBufferRegistry.get_instance().finalize(); odc.finalize_distributed(); print('ok')",
    ])
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and "ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]
