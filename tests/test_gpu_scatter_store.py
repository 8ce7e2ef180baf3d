"""The store form of scatter-accumulate (first accumulate after a clear, without the clear) and
the lazy clear built on it: the bits must be those of ``acc.fill_(0)`` followed by ``acc.add_``
(odc/primitives/scatter_accumulate.py:585-587, :386), and the accumulation must not be read."""

import ctypes
import random

import pytest
import torch

from helpers import assert_bit_equal
from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu

PAIRS = [(torch.bfloat16, torch.float32), (torch.float32, torch.float32), (torch.float16, torch.float32),
         (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.float32, torch.bfloat16),
         (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16), (torch.float32, torch.float16)]


def poison(acc_peers):
    """Fill accumulations with NaN bit patterns: any read of them would show in the result."""
    for peer in acc_peers:
        peer.view(torch.uint8).fill_(0xFF)


@pytest.mark.parametrize("grad_dtype,acc_dtype", PAIRS)
@pytest.mark.parametrize("W,S,valid_short", [(1, 5, 0), (4, 1, 1), (8, 4096, 0), (8, 4099, 13), (12, 33_337, 40_000),
                                             (3, 70_001, 3)])
def test_scatter_store_through_the_c_abi(make_world, grad_dtype, acc_dtype, W, S, valid_short):
    """odc_scatter_store over poisoned accumulations equals zeros + one oracle accumulate; the
    bytes around the accumulation slices stay as they were."""
    from odc_amd import SymmBufferRegistry, _native
    from odc_amd.primitives.utils import get_world, native_dtype

    make_world(W, 4 << 20)
    registry = SymmBufferRegistry.get_instance()
    guard = 7  # elements kept on both sides of the slice the store writes
    registry.allocate_symm_buffer("acc", (S + 2 * guard,), acc_dtype)
    peers = registry.peer_tensors["acc"]
    poison(peers)
    offset = registry.get_offset("acc") + guard * acc_dtype.itemsize
    g = torch.Generator().manual_seed(S + W)
    valid = max(0, W * S - valid_short)
    grad = torch.randn(valid + 3, generator=g).to(grad_dtype)
    grad[::5] = -0.0
    dev = grad.cuda()[3:]  # an odd element offset on the gradient side too
    assert dev.numel() == valid
    item = _native.AccumItem(dev.data_ptr(), valid, offset, S)
    items = (_native.AccumItem * 1)(item)
    _native.check(_native.load().odc_scatter_store(
        get_world().arena.handle, items, 1, native_dtype(grad_dtype), native_dtype(acc_dtype),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    host = grad[3:]
    padded = torch.cat([host, torch.zeros(W * S - host.numel(), dtype=grad_dtype)])
    want = [torch.zeros(S, dtype=acc_dtype) for _ in range(W)]
    oracle.scatter_accumulate(want, padded)
    for r, peer in enumerate(peers):
        got = peer.cpu()
        assert_bit_equal(got[guard : guard + S], want[r], f"{grad_dtype}->{acc_dtype} W={W} S={S} rank {r}")
        assert not torch.signbit(got[guard : guard + S][want[r] == 0]).any()
        edges = torch.cat([got[:guard], got[guard + S :]]).view(torch.uint8)
        assert (edges == 0xFF).all(), "bytes outside the slice were written"


def test_scatter_store_every_bf16_pattern(make_world):
    """+0 + g for every bf16 bit pattern g: -0 becomes +0, NaNs stay NaN, all else is g widened."""
    from odc_amd import ReductionService

    W = 4
    group = make_world(W, 4 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=True)
    all_bf16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    red.register("all", (65536 // W,), torch.bfloat16, torch.float32, group)
    red.clear_accumulations()  # lazy: nothing is launched, the next accumulate stores
    assert red._owed_zero == {"all"}
    poison(red._registry_peers("all"))
    red.scatter_accumulate("all", all_bf16.cuda(), group)
    want = [torch.zeros(65536 // W) for _ in range(W)]
    oracle.scatter_accumulate(want, all_bf16)
    for r, acc in enumerate(red.get_peer_accumulations("all")):
        got, w = acc.cpu(), want[r]
        nan = torch.isnan(w)
        assert torch.equal(torch.isnan(got), nan)
        assert_bit_equal(got[~nan], w[~nan], f"rank {r}")


@pytest.mark.parametrize("seed", range(10))
def test_lazy_clear_matches_the_oracle(make_world, seed):
    """A random minibatch schedule (clears, multi-key launches with repeated and missing keys,
    reads in between) under lazy clears matches the oracle, which clears eagerly; the
    accumulations are poisoned behind the service's back after every clear the service skips."""
    from odc_amd import ReductionService

    rng = random.Random(seed)
    W = rng.choice([1, 2, 4, 8, 12])
    grad_dtype, acc_dtype = PAIRS[seed % 6]
    sizes = {k: rng.choice([1, 63, 512, 4096, 4099, 20_001]) for k in "abcde"}
    group = make_world(W, 16 << 20)
    lazy = ReductionService(accumulation_dtype=acc_dtype, lazy_clear=True)
    g = torch.Generator().manual_seed(seed)
    want = {k: [torch.zeros(s, dtype=acc_dtype) for _ in range(W)] for k, s in sizes.items()}
    for k, s in sizes.items():
        lazy.register(k, (s,), grad_dtype, acc_dtype, group)
    assert not lazy._owed_zero  # registration zeroes eagerly
    for minibatch in range(3):
        lazy.clear_accumulations()
        assert lazy._owed_zero == set(sizes)
        for k in sizes:
            poison(lazy._registry_peers(k))
            for w in want[k]:
                w.zero_()
        for _ in range(rng.randrange(1, 5)):
            keys = [rng.choice("abcde") for _ in range(rng.randrange(1, 5))]
            if rng.random() < 0.5:
                keys = list(dict.fromkeys(keys))  # half of the launches without repeated keys
            grads = [torch.randn(W * sizes[k], generator=g).to(grad_dtype) for k in keys]
            lazy.scatter_accumulate_multi(keys, [x.cuda() for x in grads], group)
            for k, x in zip(keys, grads):
                oracle.scatter_accumulate(want[k], x)
            if rng.random() < 0.3:  # a read in the middle of the minibatch
                k = rng.choice("abcde")
                for r, acc in enumerate(lazy.get_peer_accumulations(k)):
                    assert_bit_equal(acc, want[k][r], f"seed {seed}: mid-minibatch read of {k} rank {r}")
        lazy.sync(group)
        for k in sizes:  # includes keys no launch touched: they must read as zeros
            for r, acc in enumerate(lazy.get_peer_accumulations(k)):
                assert_bit_equal(acc, want[k][r], f"seed {seed}: minibatch {minibatch} key {k} rank {r}")
        assert not lazy._owed_zero


@pytest.mark.parametrize("seed", range(6))
def test_slices_that_tile_the_accumulation_take_the_store_form(make_world, seed):
    """FSDP2's group layout: the per-parameter slices cover the accumulation (odd seeds: all of
    it but a gap, as the tile-aligned layout leaves them), so the first reduce of a minibatch
    needs no clear: stale sums under the slices are overwritten, the gap still holds the zeros
    of the registration."""
    from odc_amd import ReductionService

    rng = random.Random(50 + seed)
    W = rng.choice([2, 8, 12])
    grad_dtype, acc_dtype = PAIRS[seed % 3]
    sizes = [rng.choice([1, 3, 17, 1000, 4096, 4101, 30_001]) for _ in range(rng.choice([1, 4, 9, 35, 67]))]
    gap = seed % 2  # odd seeds leave one element uncovered
    offs, cur = [], 0
    for i, s in enumerate(sizes):
        if gap and i == len(sizes) // 2:
            cur += 1
        offs.append(cur)
        cur += s
    total = cur
    group = make_world(W, 16 << 20)
    red = ReductionService(accumulation_dtype=acc_dtype, lazy_clear=True)
    forms = []
    launch = red._launch
    red._launch = lambda keys, items, n, gc, ac, store: (forms.append(store), launch(keys, items, n, gc, ac, store))[1]
    g = torch.Generator().manual_seed(seed)
    want = [torch.zeros(total, dtype=acc_dtype) for _ in range(W)]
    order = list(range(len(sizes)))

    def reduce_once():
        rng.shuffle(order)  # slice order in the call is free
        valid = [rng.choice([W * s, rng.randrange(0, W * s + 1)]) for s in sizes]
        host = [torch.randn(v, generator=g).to(grad_dtype) for v in valid]
        red.scatter_accumulate_slices("g", [host[i].cuda() for i in order], [offs[i] for i in order],
                                      [sizes[i] for i in order], group, accumulation_numel=total)
        for hg, o, s in zip(host, offs, sizes):
            padded = torch.cat([hg, torch.zeros(W * s - hg.numel(), dtype=grad_dtype)])
            oracle.scatter_accumulate([w[o : o + s] for w in want], padded)

    reduce_once()  # a first minibatch: registers the accumulation (zeroed) and adds into it
    red.clear_accumulations()  # lazy: "g" now owes its zeros
    for w in want:
        w.zero_()
    for peer in red._registry_peers("g"):  # stale bytes wherever earlier launches could have left them
        for o, s in zip(offs, sizes):
            peer[o : o + s].view(torch.uint8).fill_(0xFF)
    reduce_once()
    reduce_once()
    assert forms == [False, True, False]  # after the lazy clear: one store, then adds
    for r, acc in enumerate(red.get_peer_accumulations("g")):
        assert_bit_equal(acc, want[r], f"seed {seed}: W={W} rank {r} sizes {sizes} gap {gap}")


def test_store_form_over_slices_needs_the_rest_of_the_accumulation_to_be_zero(make_world):
    """Slices with gaps between them: the lazy clear is folded into a store only while nothing
    but those slices has been written since the accumulation was last zeroed as a whole.
    Another slice layout, or a whole-key accumulate, makes the next lazy clear a real one."""
    from odc_amd import ReductionService

    W, total = 4, 20_000
    offs, sizes = [0, 4096, 12_288], [100, 5000, 4096]  # gaps after every slice
    other_offs, other_sizes = [50, 9000], [200, 1000]   # another layout: overlaps the gaps of the first
    group = make_world(W, 8 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=True)
    forms = []
    launch = red._launch
    red._launch = lambda keys, items, n, gc, ac, store: (forms.append(store), launch(keys, items, n, gc, ac, store))[1]
    g = torch.Generator().manual_seed(0)
    want = [torch.zeros(total) for _ in range(W)]

    def reduce_slices(o_list, s_list):
        host = [torch.randn(W * s, generator=g).bfloat16() for s in s_list]
        red.scatter_accumulate_slices("g", [h.cuda() for h in host], o_list, s_list, group, accumulation_numel=total)
        for h, o, s in zip(host, o_list, s_list):
            oracle.scatter_accumulate([w[o : o + s] for w in want], h)

    def new_minibatch():
        red.clear_accumulations()
        for w in want:
            w.zero_()

    def check(msg):
        # the memory as it is (nothing is owed at the points checked); a public hand-out would
        # count as a possible write between the slices, which the last part of the test covers
        assert "g" not in red._owed_zero
        for r, acc in enumerate(red._registry_peers("g")):
            assert_bit_equal(acc, want[r], f"{msg}: rank {r}")

    reduce_slices(offs, sizes)          # registers (zeroed): read-modify-write
    new_minibatch()
    reduce_slices(offs, sizes)          # only this layout written so far: store
    reduce_slices(offs, sizes)
    assert forms == [False, True, False]
    check("same layout")
    new_minibatch()                     # (check() settled nothing: nothing was owed)
    reduce_slices(other_offs, other_sizes)  # another layout while zeros are owed: real clear, then add
    assert forms[3:] == [False]
    check("other layout")
    new_minibatch()
    reduce_slices(offs, sizes)          # the other layout's data lies in this layout's gaps: real clear
    assert forms[4:] == [False]
    check("back to the first layout after a mixed minibatch")
    new_minibatch()
    reduce_slices(offs, sizes)          # that clear was a whole one and only this layout followed: store
    assert forms[5:] == [True]
    check("first layout again")
    new_minibatch()
    whole = torch.randn(W * total, generator=g).bfloat16()
    red.scatter_accumulate("g", whole.cuda(), group)  # whole key: takes the store form itself ...
    oracle.scatter_accumulate(want, whole)
    assert forms[6:] == [True]
    check("whole key")
    new_minibatch()
    reduce_slices(offs, sizes)          # ... and leaves data between the slices: real clear
    assert forms[7:] == [False]
    check("slices after a whole-key minibatch")
    new_minibatch()
    reduce_slices(offs, sizes)          # whole clear, this layout only: store
    assert forms[8:] == [True]
    # a live accumulation handed out with the promise to stay inside the slices keeps the store form
    red.get_accumulation("g", within_slices=True)[offs[1] : offs[1] + 3].add_(1.0)
    for w in want[:1]:
        w[offs[1] : offs[1] + 3] += 1.0
    check("written inside a slice through the live tensor")
    new_minibatch()
    reduce_slices(offs, sizes)
    assert forms[9:] == [True]
    # handed out without the promise, the holder may write between the slices: the next lazy
    # clear is a real one, and what was written into the gap is gone after it
    red.get_accumulation("g")[offs[0] + sizes[0] + 5] = 3.0
    new_minibatch()
    reduce_slices(offs, sizes)
    assert forms[10:] == [False]
    check("after an untracked write into a gap")


def test_clear_stays_eager_under_graph_capture(make_world):
    """A captured clear must be a kernel in the graph (a lazy clear would be host state only):
    replaying [clear] alone zeroes the accumulations every time."""
    from odc_amd import ReductionService

    W, S = 4, 10_001
    group = make_world(W, 4 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=True)
    grad = torch.ones(W * S, dtype=torch.bfloat16, device="cuda")
    red.scatter_accumulate("k", grad, group)
    red.sync(group)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        red.clear_accumulations()
    assert not red._owed_zero
    for replay in range(3):
        red.scatter_accumulate("k", grad, group)
        red.scatter_accumulate("k", grad, group)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for acc in red.get_peer_accumulations("k"):
            assert_bit_equal(acc, torch.zeros(S), f"replay {replay}")
        red.scatter_accumulate("k", grad, group)
        for acc in red.get_peer_accumulations("k"):
            assert_bit_equal(acc, torch.ones(S), f"replay {replay}: one accumulate after the clear")


@pytest.mark.parametrize("lazy", [True, False])
def test_captured_accumulate_with_clears_outside_the_graph(make_world, lazy):
    """A graph that holds only the scatter-accumulate, replayed M times per minibatch, with
    clear_accumulations() called OUTSIDE capture between minibatches: the graph always replays
    the read-modify-write form, so the clear must be a kernel even in lazy mode, and a later
    get_accumulation must not zero what the replays added."""
    from odc_amd import ReductionService

    W, S, M = 4, 30_001, 3
    group = make_world(W, 8 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    g = torch.Generator().manual_seed(21)
    grad_host = (torch.randn(W * S, generator=g) * 1e-3).bfloat16()
    grad = grad_host.cuda()
    eager_host = (torch.randn(W * S, generator=g) * 1e-3).bfloat16()
    # warm-up as torch's graph recipe has it: one eager call (registers the key, takes the store
    # form in lazy mode), then the capture
    red.clear_accumulations()
    red.scatter_accumulate("k", grad, group)
    red.sync(group)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        red.scatter_accumulate("k", grad, group)
    for minibatch in range(2):
        red.clear_accumulations()  # outside capture
        want = [torch.zeros(S) for _ in range(W)]
        for m in range(M):
            graph.replay()
            oracle.scatter_accumulate(want, grad_host)
            if m == 0:  # eager work of the same key between replays
                red.scatter_accumulate("k", eager_host.cuda(), group)
                oracle.scatter_accumulate(want, eager_host)
            torch.cuda.synchronize()
        for r, acc in enumerate(red.get_peer_accumulations("k")):
            assert_bit_equal(acc, want[r], f"minibatch {minibatch}, rank {r}")
        assert_bit_equal(red.get_accumulation("k"), want[0], f"minibatch {minibatch}: handed out")


def test_capture_refuses_an_accumulation_that_owes_zeros(make_world):
    """Lazy mode: recording the store form (or a clear) into a graph would overwrite the sums on
    every replay, so a capture that meets owed zeros fails loudly instead."""
    from odc_amd import ReductionService

    W, S = 4, 4096
    group = make_world(W, 4 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=True)
    grad = torch.ones(W * S, dtype=torch.bfloat16, device="cuda")
    red.scatter_accumulate("k", grad, group)
    red.clear_accumulations()  # "k" now owes zeros
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="owe the zeros"):
        with torch.cuda.graph(graph):
            red.scatter_accumulate("k", grad, group)
    torch.cuda.synchronize()
    # registering under capture is refused as well (its zeroing would be recorded)
    graph2 = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="before capturing"):
        with torch.cuda.graph(graph2):
            red.scatter_accumulate("new", grad, group)
    torch.cuda.synchronize()
    # the service still works eagerly afterwards
    red.scatter_accumulate("k", grad, group)
    assert_bit_equal(red.get_accumulation("k"), torch.ones(S), "store after the refused capture")


@pytest.mark.parametrize("lazy", [True, False])
def test_captured_minibatch_folds_the_clear_into_the_first_accumulate(make_world, lazy):
    """One graph = one whole minibatch: clear_accumulations() + M x scatter-accumulate, captured
    inside captured_minibatch(). The captured clear records no kernel for the keys the graph
    accumulates into (their first accumulate is the store form) and a real clear for the key it
    never touches. Replayed over 3 minibatches with every accumulation poisoned in between (a
    read-modify-write of the first microbatch, or a missing clear, would show the poison), and
    with eager work between the replays; every replay is bit-exact against the oracle."""
    from odc_amd import ReductionService

    W, M = 4, 8
    sizes = {"a": 30_001, "b": 4096, "c": 7, "idle": 5_000}
    group = make_world(W, 8 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    g = torch.Generator().manual_seed(77)
    keys = ["a", "b", "c"]
    host = [[(torch.randn(W * sizes[k], generator=g) * 1e-3).bfloat16() for k in keys] for _ in range(M)]
    for mb in host:
        mb[0][::3] = -0.0  # a store that copied instead of adding +0 would leave -0
    dev = [[t.cuda() for t in mb] for mb in host]
    for k, n in sizes.items():
        red.register(k, (n,), torch.bfloat16, torch.float32, group)
    # one eager minibatch first (torch's capture recipe warms up eagerly)
    red.clear_accumulations()
    for m in range(M):
        red.scatter_accumulate_multi(keys, dev[m], group)
    red.sync(group)
    for k in sizes:
        red.get_accumulation(k)  # settles whatever a lazy clear still owes
    torch.cuda.synchronize()

    launches = []
    real_launch = red._launch
    real_clear = red._clear_keys

    def spy_launch(keys_, items, n, grad_code, acc_code, store):
        launches.append(("store" if store else "rmw", tuple(keys_)))
        return real_launch(keys_, items, n, grad_code, acc_code, store)

    def spy_clear(keys_):
        keys_ = list(keys_)
        if keys_:
            launches.append(("clear", tuple(keys_)))
        return real_clear(keys_)

    red._launch, red._clear_keys = spy_launch, spy_clear
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), red.captured_minibatch():
        red.clear_accumulations()
        for m in range(M):
            red.scatter_accumulate_multi(keys, dev[m], group)
    red._launch, red._clear_keys = real_launch, real_clear
    assert launches[0] == ("store", ("a", "b", "c")), launches[:2]
    assert launches[1:M] == [("rmw", ("a", "b", "c"))] * (M - 1)
    assert launches[M:] == [("clear", ("idle",))], "the key the graph never accumulates into is cleared by a kernel"

    want = {k: [torch.zeros(sizes[k]) for _ in range(W)] for k in keys}
    for m in range(M):
        for k, t in zip(keys, host[m]):
            oracle.scatter_accumulate(want[k], t)
    for replay in range(3):
        for k in sizes:
            poison(red._registry_peers(k))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k in keys:
            for r, acc in enumerate(red._registry_peers(k)):
                assert_bit_equal(acc, want[k][r], f"replay {replay}, key {k}, rank {r}")
        for acc in red._registry_peers("idle"):
            assert_bit_equal(acc, torch.zeros(sizes["idle"]), f"replay {replay}: idle key cleared")
        # the program's own eager work between replays: one more accumulate, read-modify-write
        red.scatter_accumulate("b", dev[0][1], group)
        torch.cuda.synchronize()
        extra = [w.clone() for w in want["b"]]
        oracle.scatter_accumulate(extra, host[0][1])
        for r, acc in enumerate(red.get_peer_accumulations("b")):
            assert_bit_equal(acc, extra[r], f"replay {replay}: eager accumulate after the replay")
    # an eager clear outside capture still zeroes the captured keys with a kernel, lazy or not
    red.clear_accumulations()
    torch.cuda.synchronize()
    for k in keys:
        for acc in red._registry_peers(k):
            assert_bit_equal(acc, torch.zeros(sizes[k]), "eager clear of a captured key")


def test_captured_minibatch_settles_reads_and_gapped_slices(make_world):
    """Inside captured_minibatch(): a key that is published before its first accumulate gets
    its clear recorded in front of the publish; slices with gaps get a real clear (what lies
    between them at replay time is unknown), slices that tile the accumulation take the store
    form; and a block outside capture, or nested, is refused."""
    from odc_amd import ReductionService

    W = 4
    group = make_world(W, 8 << 20)
    red = ReductionService(accumulation_dtype=torch.float32)
    with pytest.raises(RuntimeError, match="inside torch.cuda.graph"):
        with red.captured_minibatch():
            pass
    sizes, gapped, tiled = [5000, 300], [0, 8192], [0, 5000]
    g = torch.Generator().manual_seed(5)
    host = [(torch.randn(W * n, generator=g) * 1e-3).bfloat16() for n in sizes]
    dev = [t.cuda() for t in host]
    red.register("read", (64,), torch.bfloat16, torch.float32, group)
    red.scatter_accumulate_slices("gapped", dev, gapped, sizes, group, accumulation_numel=8192 + 300)
    red.scatter_accumulate_slices("tiled", dev, tiled, sizes, group, accumulation_numel=5300)
    red.sync(group)
    torch.cuda.synchronize()
    forms = []
    real_launch, real_clear = red._launch, red._clear_keys
    red._launch = lambda k, i, n, gc_, ac, store: (forms.append(("store" if store else "rmw", tuple(k))),
                                                     real_launch(k, i, n, gc_, ac, store))[1]
    red._clear_keys = lambda k: (forms.append(("clear", tuple(k))) if list(k) else None, real_clear(k))[1]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), red.captured_minibatch():
        with pytest.raises(RuntimeError, match="do not nest"):
            with red.captured_minibatch():
                pass
    graph = torch.cuda.CUDAGraph()
    forms.clear()
    with torch.cuda.graph(graph), red.captured_minibatch():
        red.clear_accumulations()
        out = red.publish(["read"], out_dtype=torch.bfloat16)[0]
        red.scatter_accumulate_slices("gapped", dev, gapped, sizes, group)
        red.scatter_accumulate_slices("tiled", dev, tiled, sizes, group)
        red.scatter_accumulate_slices("tiled", dev, tiled, sizes, group)
    red._launch, red._clear_keys = real_launch, real_clear
    assert forms == [("clear", ("read",)), ("clear", ("gapped",)), ("rmw", ("gapped",)), ("store", ("tiled",)),
                     ("rmw", ("tiled",))], forms
    for replay in range(2):
        for k in ("read", "gapped", "tiled"):
            poison(red._registry_peers(k))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bit_equal(out, torch.zeros(64, dtype=torch.bfloat16), "published zeros")
        for r in range(W):
            want_g, want_t = torch.zeros(8192 + 300), torch.zeros(5300)
            for off_g, off_t, n, t in zip(gapped, tiled, sizes, host):
                chunk = t.view(W, n)[r].float()
                want_g[off_g : off_g + n] += chunk
                want_t[off_t : off_t + n] += chunk
                want_t[off_t : off_t + n] += chunk
            assert_bit_equal(red._registry_peers("gapped")[r], want_g, f"replay {replay} gapped rank {r}")
            assert_bit_equal(red._registry_peers("tiled")[r], want_t, f"replay {replay} tiled rank {r}")
