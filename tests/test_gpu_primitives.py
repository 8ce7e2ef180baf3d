"""GPU parity of the two primitives against the CPU oracle, through the Python mirror of the
reference API (which calls the C ABI of libodc_hip.so). Bit-exact: gather is a byte copy;
scatter-accumulate does one IEEE fp32 add per element per call, in call order."""


import pytest
import torch

from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu


from helpers import assert_bit_equal


def services():
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry

    return GatherService(), ReductionService(accumulation_dtype=torch.float32), SymmBufferRegistry.get_instance()


def put_shards(registry, key, shards, group):
    from helpers import put_shards as _put

    return _put(registry, key, shards)


def test_gather_known_answer_pattern(make_world):
    """examples/all_gather.py:80-84,121-125: tensor i on rank r is filled with i + 2r; block r of
    the gathered tensor must equal 2r + i exactly (int64 there and here)."""
    W, size, cnt = 8, 1 << 16, 5
    group = make_world(W, 64 << 20)
    gather, _, registry = services()
    for i in range(cnt):
        shards = [torch.full((size,), i + 2 * r, dtype=torch.int64) for r in range(W)]
        src = put_shards(registry, i, shards, group)
        dst = torch.empty(size * W, dtype=torch.int64, device="cuda")
        gather.gather_into_tensor(dst, src, group)
        for r in range(W):
            assert torch.eq(dst[r * size : (r + 1) * size], 2 * r + i).all()


def test_config1_plumbing(make_world):
    """W=4, one flat bf16 param of 4 Mi elements N(0, 0.02) seed 0 in 4 equal shards, gathered;
    then 4 microbatches of bf16 grads N(0, 1e-3) scatter-accumulated into zeroed fp32 shards."""
    W, N, M = 4, 4_194_304, 4
    g = torch.Generator().manual_seed(0)
    param = (torch.randn(N, generator=g) * 0.02).bfloat16()
    grads = [(torch.randn(N, generator=g) * 1e-3).bfloat16() for _ in range(M)]
    shards = list(param.view(W, -1))

    group = make_world(W, 64 << 20)
    gather, reduction, registry = services()
    src = put_shards(registry, "flat", shards, group)
    out = torch.empty(N, dtype=torch.bfloat16, device="cuda")
    gather.gather_into_tensor(out, src, group)
    assert_bit_equal(out, oracle.gather(shards), "gather")
    assert_bit_equal(out, param, "gather vs original")

    want = [torch.zeros(N // W, dtype=torch.float32) for _ in range(W)]
    reduction.clear_accumulations()
    for m in range(M):
        reduction.scatter_accumulate("flat", grads[m].cuda(), group)
        oracle.scatter_accumulate(want, grads[m])
    reduction.sync(group)
    for r, acc in enumerate(reduction.get_peer_accumulations("flat")):
        assert_bit_equal(acc, want[r], f"accumulation of rank {r}")
    # clear brings every rank back to +0.0
    reduction.clear_accumulations()
    reduction.sync(group)
    for acc in reduction.get_peer_accumulations("flat"):
        assert_bit_equal(acc, torch.zeros(N // W), "cleared accumulation")


@pytest.mark.parametrize("W", [1, 2, 3, 5, 8, 12, 64, 200])
@pytest.mark.parametrize("S", [0, 1, 7, 63, 64, 65, 4095, 4096, 4097, 16384 + 3, 100_003])
def test_gather_any_shard_size(make_world, W, S):
    """Byte copy at every alignment: odd shard sizes put block r of the output at odd offsets."""
    group = make_world(W, 4 << 20)
    gather, _, registry = services()
    g = torch.Generator().manual_seed(W * 1000 + S)
    shards = [torch.randint(-32768, 32767, (S,), generator=g, dtype=torch.int16) for _ in range(W)]
    src = put_shards(registry, "p", shards, group)
    # sentinels on both sides of the destination catch writes outside [0, W*S)
    pad = 64
    buf = torch.full((W * S + 2 * pad,), -999, dtype=torch.int16, device="cuda")
    dst = buf[pad : pad + W * S]
    from odc_amd import virtual_rank

    with virtual_rank(W - 1):  # rotation start must not matter (gather.py:122)
        gather.gather_into_tensor(dst, registry.get_symm_buffer("p"), group)
    assert_bit_equal(dst, oracle.gather(shards), f"W={W} S={S}")
    assert (buf[:pad] == -999).all() and (buf[pad + W * S :] == -999).all()


@pytest.mark.parametrize("grad_dtype,acc_dtype", [
    (torch.bfloat16, torch.float32),
    (torch.float32, torch.float32),
    (torch.float16, torch.float32),
    (torch.bfloat16, torch.bfloat16),
    (torch.float16, torch.float16),
])
@pytest.mark.parametrize("W,S", [(1, 5), (4, 1), (8, 4096), (8, 4099), (12, 33_337), (3, 70_001), (200, 4_101)])
def test_scatter_accumulate_dtypes_and_sizes(make_world, grad_dtype, acc_dtype, W, S):
    from odc_amd import ReductionService

    group = make_world(W, 4 << 20)
    reduction = ReductionService(accumulation_dtype=acc_dtype)
    g = torch.Generator().manual_seed(S)
    want = [torch.zeros(S, dtype=acc_dtype) for _ in range(W)]
    for m in range(3):
        grad = torch.randn(W * S, generator=g).to(grad_dtype)
        reduction.scatter_accumulate(7, grad.cuda(), group)
        oracle.scatter_accumulate(want, grad)
    reduction.sync(group)
    for r, acc in enumerate(reduction.get_peer_accumulations(7)):
        assert_bit_equal(acc, want[r], f"{grad_dtype}->{acc_dtype} W={W} S={S} rank {r}")


def test_scatter_accumulate_special_values(make_world):
    """Signed zero (+0 + -0 = +0), denormals, infinities, NaN propagation, bf16 extremes."""
    W = 4
    group = make_world(W, 4 << 20)
    from odc_amd import ReductionService

    reduction = ReductionService(accumulation_dtype=torch.float32)
    # every bf16 bit pattern once, as the gradient
    all_bf16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    assert all_bf16.numel() % W == 0
    want = [torch.zeros(all_bf16.numel() // W) for _ in range(W)]
    for _ in range(2):
        reduction.scatter_accumulate("all", all_bf16.cuda(), group)
        oracle.scatter_accumulate(want, all_bf16)
    reduction.sync(group)
    for r, acc in enumerate(reduction.get_peer_accumulations("all")):
        got, w = acc.cpu(), want[r]
        nan = torch.isnan(w)
        assert torch.equal(torch.isnan(got), nan)
        assert_bit_equal(got[~nan], w[~nan], f"rank {r}")
    # -0 gradients into a cleared (+0) accumulation give +0, not -0
    neg0 = torch.full((W * 8,), -0.0).bfloat16()
    reduction.scatter_accumulate("z", neg0.cuda(), group)
    reduction.sync(group)
    for acc in reduction.get_peer_accumulations("z"):
        assert not torch.signbit(acc.cpu()).any()
    # fp32 denormals survive (no flush to zero)
    tiny = torch.full((W * 8,), 1e-41, dtype=torch.float32)
    reduction.scatter_accumulate("d", tiny.cuda(), group)
    reduction.scatter_accumulate("d", tiny.cuda(), group)
    reduction.sync(group)
    wantd = [torch.zeros(8) for _ in range(W)]
    oracle.scatter_accumulate(wantd, tiny)
    oracle.scatter_accumulate(wantd, tiny)
    for r, acc in enumerate(reduction.get_peer_accumulations("d")):
        assert_bit_equal(acc, wantd[r], "denormal")
        assert (acc.cpu() != 0).all()


def test_hip_graph_capture_and_replay(make_world):
    """No entry point allocates, synchronises or memsets, so clear + scatter-accumulate + gather
    can be captured in a HIP graph; every replay (with eager work and synchronisations between
    replays) must reproduce the eager result."""
    from odc_amd import virtual_rank

    W, S = 8, 50_003
    group = make_world(W, 16 << 20)
    gather, reduction, registry = services()
    g = torch.Generator().manual_seed(9)
    shards = [(torch.randn(S, generator=g) * 0.02).bfloat16() for _ in range(W)]
    src = put_shards(registry, "p", shards, group)
    grad = (torch.randn(W * S, generator=g) * 1e-3).bfloat16().cuda()
    grad2 = (torch.randn(W * S, generator=g) * 1e-3).bfloat16()
    out = torch.zeros(W * S, dtype=torch.bfloat16, device="cuda")
    reduction.register("p", (S,), torch.bfloat16, torch.float32, group)
    reduction.sync(group)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        reduction.clear_accumulations()
        reduction.scatter_accumulate("p", grad, group)
        reduction.scatter_accumulate("p", grad, group)
        gather.gather_into_tensor(out, src, group)
    want_acc = [torch.zeros(S) for _ in range(W)]
    oracle.scatter_accumulate(want_acc, grad.cpu())
    oracle.scatter_accumulate(want_acc, grad.cpu())
    for replay in range(4):
        # eager work between replays: dirty the outputs, move the inputs' values
        out.fill_(7.0)
        reduction.scatter_accumulate("p", grad2.cuda(), group)
        with virtual_rank(replay % W):
            registry.get_symm_buffer("p").add_(1.0)
        shards[replay % W] = (shards[replay % W].float() + 1.0).bfloat16()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bit_equal(out, oracle.gather(shards), f"replay {replay}: gather")
        for r, acc in enumerate(reduction.get_peer_accumulations("p")):
            assert_bit_equal(acc, want_acc[r], f"replay {replay}: accumulation of rank {r}")


@pytest.mark.parametrize("src_dtype,dst_dtype", [
    (torch.float32, torch.bfloat16), (torch.float32, torch.float16), (torch.bfloat16, torch.float32),
    (torch.float16, torch.float32), (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16),
])
@pytest.mark.parametrize("W,S", [(1, 3), (8, 4096), (8, 4099), (12, 33_337), (3, 70_001), (64, 64)])
def test_gather_with_cast(make_world, src_dtype, dst_dtype, W, S):
    """Shards in one dtype gathered into a full parameter of another in one pass equal the
    reference's gather-then-cast."""
    group = make_world(W, 4 << 20)
    gather, _, registry = services()
    g = torch.Generator().manual_seed(S + W)
    shards = [(torch.randn(S, generator=g) * 10.0 ** (r % 5 - 2)).to(src_dtype) for r in range(W)]
    src = put_shards(registry, "p", shards, group)
    buf = torch.full((W * S + 16,), 7.0, dtype=dst_dtype, device="cuda")
    dst = buf[5 : 5 + W * S]  # odd element offset: unaligned destination
    gather.gather_into_tensor(dst, src, group)
    assert_bit_equal(dst, oracle.gather_cast(shards, dst_dtype), f"{src_dtype}->{dst_dtype} W={W} S={S}")
    assert (buf[:5] == 7).all() and (buf[5 + W * S :] == 7).all()


ALL_PAIRS = [(a, b) for a in (torch.float32, torch.bfloat16, torch.float16)
             for b in (torch.float32, torch.bfloat16, torch.float16)]


@pytest.mark.parametrize("src_dtype,dst_dtype", ALL_PAIRS)
@pytest.mark.parametrize("W,n,lead", [(1, 3, 0), (8, 4096, 0), (8, 4099, 3), (12, 33_337, 1), (3, 70_001, 5), (64, 64, 0)])
def test_convert_all_ranks_in_one_launch(make_world, src_dtype, dst_dtype, W, n, lead):
    """odc_convert through the C ABI: every rank's slice of one symmetric buffer converted into
    that rank's slice of another, in one launch, equals torch's CPU ``.to(dtype)`` (round to
    nearest even) per rank; the elements around the destination slices keep their values. Equal
    dtypes make it a symmetric copy."""
    import ctypes

    from odc_amd import _native
    from odc_amd.primitives.utils import get_world, native_dtype

    make_world(W, 4 << 20)
    _, _, registry = services()
    guard = 9
    registry.allocate_symm_buffer("src", (n + lead,), src_dtype)
    registry.allocate_symm_buffer("dst", (n + lead + 2 * guard,), dst_dtype)
    g = torch.Generator().manual_seed(n + W)
    shards = [(torch.randn(n + lead, generator=g) * 10.0 ** (r % 5 - 2)).to(src_dtype) for r in range(W)]
    for peer, shard in zip(registry.peer_tensors["src"], shards):
        peer.copy_(shard)
    for peer in registry.peer_tensors["dst"]:
        peer.fill_(7.0)
    item = (_native.ConvertItem * 2)()
    item[0].src_offset = registry.get_offset("src") + lead * src_dtype.itemsize
    item[0].dst_offset = registry.get_offset("dst") + (guard + lead) * dst_dtype.itemsize
    item[0].elems = n
    item[1].elems = 0  # empty items take no part
    _native.check(_native.load().odc_convert(
        get_world().arena.handle, item, 2, native_dtype(src_dtype), native_dtype(dst_dtype),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    for r, peer in enumerate(registry.peer_tensors["dst"]):
        got = peer.cpu()
        assert_bit_equal(got[guard + lead : guard + lead + n], shards[r][lead:].to(dst_dtype), f"rank {r}")
        assert (got[: guard + lead] == 7).all() and (got[guard + lead + n :] == 7).all(), f"rank {r}: guards"


def test_convert_special_values_and_errors(make_world):
    """Ties, overflow, denormals, signed zero and NaN through the one-launch conversion (fp32 ->
    bf16), and the argument checks of odc_convert."""
    import ctypes

    from odc_amd import GatherService, _native
    from odc_amd.primitives.utils import get_world

    W = 4
    make_world(W, 4 << 20)
    _, _, registry = services()
    ties = (2.0 ** torch.arange(-149, 127, dtype=torch.float64)).float() * 1.00390625
    vals = torch.cat([ties, -ties, torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 3.4e38, -3.4e38, 1e-45, float("nan")])])
    vals = torch.cat([vals, torch.zeros((-vals.numel()) % W)])
    n = vals.numel() // W
    registry.allocate_symm_buffer("m", (n,), torch.float32)
    registry.allocate_symm_buffer("c", (n,), torch.bfloat16)
    for peer, shard in zip(registry.peer_tensors["m"], vals.view(W, -1)):
        peer.copy_(shard)
    GatherService().convert_symm_buffer("c", "m")
    torch.cuda.synchronize()
    got = torch.cat([p.cpu() for p in registry.peer_tensors["c"]])
    want = vals.bfloat16()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    assert_bit_equal(got[~nan], want[~nan], "ties, overflow to inf, denormals, signed zero")

    lib, arena = _native.load(), get_world().arena.handle
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    src, dst = registry.get_offset("m"), registry.get_offset("c")

    def status(src_offset, dst_offset, elems, sd=_native.DTYPE_F32, dd=_native.DTYPE_BF16):
        item = (_native.ConvertItem * 1)()
        item[0].src_offset, item[0].dst_offset, item[0].elems = src_offset, dst_offset, elems
        return lib.odc_convert(arena, item, 1, sd, dd, stream)

    assert status(src, dst, n) == _native.ODC_OK
    assert status(src + 2, dst, n - 1) == _native.ODC_ERR_INVALID  # source not fp32 aligned
    assert status(src, dst + 1, n - 1) == _native.ODC_ERR_INVALID  # destination not bf16 aligned
    assert status(src, src + 4, n - 1) == _native.ODC_ERR_INVALID  # overlap
    assert b"overlaps" in lib.odc_last_error()
    assert status(src, dst, 1 << 62) == _native.ODC_ERR_INVALID  # byte size would wrap
    assert status((4 << 20) - 4, dst, 2) == _native.ODC_ERR_INVALID  # leaves the rank region
    assert status(src, dst, n, sd=7) == _native.ODC_ERR_INVALID  # unknown dtype code
    assert lib.odc_convert(arena, None, 1, _native.DTYPE_F32, _native.DTYPE_BF16, stream) == _native.ODC_ERR_INVALID
    torch.cuda.synchronize()


def test_gather_with_cast_special_values(make_world):
    W = 4
    group = make_world(W, 4 << 20)
    gather, _, registry = services()
    ties = (2.0 ** torch.arange(-149, 127, dtype=torch.float64)).float() * 1.00390625
    vals = torch.cat([ties, -ties, torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 3.4e38, -3.4e38, 1e-45, float("nan")])])
    vals = torch.cat([vals, torch.zeros((-vals.numel()) % W)])
    shards = list(vals.view(W, -1))
    src = put_shards(registry, "v", shards, group)
    out = torch.empty(vals.numel(), dtype=torch.bfloat16, device="cuda")
    gather.gather_into_tensor(out, src, group)
    want = oracle.gather_cast(shards, torch.bfloat16)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(out.cpu()), nan)
    assert_bit_equal(out.cpu()[~nan], want[~nan], "ties, overflow to inf, denormals, signed zero")


@pytest.mark.parametrize("divisor", [1.0, 8.0, 12.0, 3.0])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_publish_divides_in_place_and_casts(make_world, divisor, out_dtype):
    """acc /= divisor with a correctly rounded division (bit-equal to torch CPU div_) and the cast
    copy, for two keys in one launch, on a rank other than 0."""
    from odc_amd import ReductionService, virtual_rank

    W = 4
    group = make_world(W, 4 << 20)
    reduction = ReductionService(accumulation_dtype=torch.float32)
    g = torch.Generator().manual_seed(int(divisor))
    sizes = {"a": 10_007, "b": 4096}
    want = {k: [torch.zeros(n) for _ in range(W)] for k, n in sizes.items()}
    for k, n in sizes.items():
        grad = torch.randn(W * n, generator=g).bfloat16()
        reduction.scatter_accumulate(k, grad.cuda(), group)
        oracle.scatter_accumulate(want[k], grad)
    with virtual_rank(2):
        outs = reduction.publish(["a", "b"], out_dtype=out_dtype, divisor=divisor)
        reduction.sync(group)
        for k, out in zip(sizes, outs):
            acc = want[k][2].clone()
            expect = oracle.fsdp1_publish(acc, divisor, out_dtype)
            assert_bit_equal(out, expect, f"published {k}")
            assert_bit_equal(reduction.get_accumulation(k), acc, f"accumulation {k} divided in place")
            if out_dtype == torch.float32:
                assert out.data_ptr() == reduction.get_accumulation(k).data_ptr()  # no copy, like .to()
    for r in (0, 1, 3):  # other ranks untouched
        assert_bit_equal(reduction.get_peer_accumulations("a")[r], want["a"][r], f"rank {r}")


def test_every_virtual_rank_as_a_client(make_world):
    """examples/reduce_scatter.py:96-105,163-172 on one GPU: each of the W ranks scatter-accumulates
    its own gradient, one after the other, for several rounds; rank r's accumulation then equals
    the reduce-scatter sum of chunk r over clients, accumulated over rounds (within the reference's
    rtol=atol=5e-3, and bit for bit equal to the oracle run in the same client order). Gathers
    issued from every rank's point of view give the same result."""
    from odc_amd import virtual_rank

    W, S, rounds = 8, 16 * 1024 + 128, 4
    group = make_world(W, 16 << 20)
    gather, reduction, registry = services()
    g = torch.Generator().manual_seed(21)
    want = [torch.zeros(S) for _ in range(W)]
    nccl_like = [torch.zeros(S) for _ in range(W)]
    for _ in range(rounds):
        client_grads = [torch.rand(W * S, generator=g) for _ in range(W)]  # fp32 grads, as the example
        for q in range(W):
            with virtual_rank(q):
                reduction.scatter_accumulate(0, client_grads[q].cuda(), group)
            oracle.scatter_accumulate(want, client_grads[q])
        reduced = torch.stack(client_grads).sum(0).view(W, S)  # reduce_scatter(SUM) ...
        for r in range(W):
            nccl_like[r].add_(reduced[r])  # ... followed by add_
    reduction.sync(group)
    for r, acc in enumerate(reduction.get_peer_accumulations(0)):
        assert_bit_equal(acc, want[r], f"rank {r}")
        torch.testing.assert_close(acc.cpu(), nccl_like[r], rtol=5e-3, atol=5e-3)
    shards = [torch.randn(S, generator=g).bfloat16() for _ in range(W)]
    put_shards(registry, "p", shards, group)
    for q in range(W):
        with virtual_rank(q):
            out = torch.empty(W * S, dtype=torch.bfloat16, device="cuda")
            gather.gather_into_tensor(out, registry.get_symm_buffer("p"), group)
            assert_bit_equal(out, oracle.gather(shards), f"gather as rank {q}")


def test_services_called_from_several_host_threads(make_world):
    """FSDP calls the primitives from the main thread (forward) and from autograd's device thread
    (backward): concurrent callers, each with keys of its own, must all get exact results."""
    import threading

    W, S, T, M = 8, 20_003, 4, 12
    group = make_world(W, 32 << 20)
    gather, reduction, registry = services()
    g = torch.Generator().manual_seed(3)
    shards = {t: [(torch.randn(S, generator=g) * 0.02).bfloat16() for _ in range(W)] for t in range(T)}
    grads = {t: [(torch.randn(W * S, generator=g) * 1e-3).bfloat16() for _ in range(M)] for t in range(T)}
    srcs = {t: put_shards(registry, ("p", t), shards[t], group) for t in range(T)}
    dev_grads = {t: [x.cuda() for x in grads[t]] for t in range(T)}
    outs = {t: torch.zeros(W * S, dtype=torch.bfloat16, device="cuda") for t in range(T)}
    for t in range(T):
        reduction.register(("k", t), (S,), torch.bfloat16, torch.float32, group)
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            torch.cuda.set_device(0)
            for m in range(M):
                gather.gather_into_tensor(outs[t], srcs[t], group)
                reduction.scatter_accumulate(("k", t), dev_grads[t][m], group)
        except Exception as e:  # noqa: BLE001 - reported on the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(T)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    reduction.sync(group)
    torch.cuda.synchronize()
    for t in range(T):
        assert_bit_equal(outs[t], oracle.gather(shards[t]), f"thread {t}: gather")
        want = [torch.zeros(S) for _ in range(W)]
        for m in range(M):
            oracle.scatter_accumulate(want, grads[t][m])
        for r, acc in enumerate(reduction.get_peer_accumulations(("k", t))):
            assert_bit_equal(acc, want[r], f"thread {t}: accumulation of rank {r}")


@pytest.mark.parametrize("policy", ["caller", "dedicated"])
def test_launch_stream_policies(make_world, monkeypatch, policy):
    """ODC_COMM_STREAM=caller launches on the caller's current stream, =dedicated hops to the one
    comm stream with joins on both sides (gather.py:114,176): either way a call is ordered like
    work on the caller's stream, from the default stream and from a side stream alike, and
    ``sync`` waits for everything launched."""
    from odc_amd.primitives import utils

    monkeypatch.setenv("ODC_COMM_STREAM", policy)
    W, S = 8, 30_011
    group = make_world(W, 16 << 20)
    gather, reduction, registry = services()
    g = torch.Generator().manual_seed(11)
    shards = [(torch.randn(S, generator=g) * 0.02).bfloat16() for _ in range(W)]
    src = put_shards(registry, "p", shards, group)
    grads = [(torch.randn(W * S, generator=g) * 1e-3).bfloat16() for _ in range(4)]
    want = [torch.zeros(S) for _ in range(W)]
    side = torch.cuda.Stream()
    out = torch.empty(W * S, dtype=torch.bfloat16, device="cuda")
    for m, grad in enumerate(grads):
        dev = grad.cuda()
        stream = side if m % 2 else torch.cuda.current_stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            src.add_(0.5)  # producer on the caller's stream right before the call
            gather.gather_into_tensor(out, src, group)
            doubled = out.float() * 2  # consumer on the caller's stream right after it
            reduction.scatter_accumulate("k", dev, group)
        torch.cuda.current_stream().wait_stream(stream)
        shards[0] = (shards[0].float() + 0.5).bfloat16()
        oracle.scatter_accumulate(want, grad)
        assert_bit_equal(doubled, oracle.gather(shards).float() * 2, f"{policy}: microbatch {m}")
    launched_on = set(utils._launch_streams)
    if policy == "dedicated":
        assert launched_on == {utils.get_comm_stream().cuda_stream}
    else:
        assert side.cuda_stream in launched_on
    reduction.sync(group)
    assert not utils._launch_streams
    for r, acc in enumerate(reduction.get_peer_accumulations("k")):
        assert_bit_equal(acc, want[r], f"{policy}: accumulation of rank {r}")
    monkeypatch.setenv("ODC_COMM_STREAM", "sideways")
    with pytest.raises(ValueError):
        gather.gather_into_tensor(out, src, group)


@pytest.mark.parametrize("store", [False, True])
def test_long_lists_mixing_tiny_and_large_items(make_world, store):
    """300 keys in ONE call, every third of less than one tile per rank (those are launched after
    the others, and a list this long takes the heap-allocated launch order and five launches):
    every key gets exactly its own gradient, twice, in the read-modify-write form and after a lazy
    clear in the store form."""
    W = 4
    group = make_world(W, 64 << 20)
    _, _, registry = services()
    from odc_amd import ReductionService

    reduction = ReductionService(accumulation_dtype=torch.float32, lazy_clear=store)
    g = torch.Generator().manual_seed(31)
    sizes = [(7 + i if i % 3 == 0 else 4096 + 17 * i) for i in range(300)]
    keys = [f"k{i}" for i in range(len(sizes))]
    grads = [(torch.randn(W * s, generator=g) * 1e-3).bfloat16() for s in sizes]
    dev = [t.cuda() for t in grads]
    for k, s in zip(keys, sizes):
        reduction.register(k, (s,), torch.bfloat16, torch.float32, group)
    reduction.clear_accumulations()
    reduction.scatter_accumulate_multi(keys, dev, group)
    reduction.scatter_accumulate_multi(keys, dev, group)
    reduction.sync(group)
    for k, s, t in zip(keys, sizes, grads):
        want = [torch.zeros(s) for _ in range(W)]
        oracle.scatter_accumulate(want, t)
        oracle.scatter_accumulate(want, t)
        for r, acc in enumerate(reduction.get_peer_accumulations(k)):
            assert_bit_equal(acc, want[r], f"key {k} rank {r}")
