"""Callers on several streams and host threads.

In the reference every add into a rank's accumulation is performed by that rank's one watcher,
in the order the requests arrive (odc/primitives/scatter_accumulate.py:291-310, :386-392), so
clients on different streams cannot race on an accumulation. Here the add is a read-modify-write
on the caller's stream; the service orders launches that touch the same key across streams. The
tests use launches long enough (tens of microseconds) to overlap if nothing ordered them."""

import threading

import pytest
import torch

from helpers import assert_bit_equal
from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu

W, S = 4, 1_500_000  # 6 M elements per launch: ~10 us of kernel, launches from idle streams overlap


def _integer_grads(n, count, gen):
    """bf16 gradients with small integer values: any order of adding them gives the same fp32
    bits, so a lost or torn update shows as a bit difference whatever the interleaving."""
    return [torch.randint(-8, 9, (n,), generator=gen).to(torch.bfloat16) for _ in range(count)]


def _run_threads(T, body):
    errors = []
    barrier = threading.Barrier(T)

    def run(t):
        try:
            barrier.wait()
            body(t)
        except BaseException as e:  # noqa: BLE001 - reported by the test below
            errors.append(e)

    threads = [threading.Thread(target=run, args=(t,)) for t in range(T)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


@pytest.mark.parametrize("lazy", [False, True])
def test_host_threads_on_streams_of_their_own_accumulate_into_one_key(make_world, lazy):
    """T host threads, each on a stream of its own, scatter-accumulate M gradients each into ONE
    key. The order between threads is free (the reference's is arrival order), so: integer-valued
    gradients must come out bit-exact whatever the order, and N(0,1e-3) gradients within the
    rtol of 1e-6 that holds for a reordered fp32 sum."""
    from odc_amd import ReductionService

    T, M = 4, 6
    group = make_world(W, 64 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    gen = torch.Generator().manual_seed(3)
    red.register("k", (S,), torch.bfloat16, torch.float32, group)
    red.register("r", (S,), torch.bfloat16, torch.float32, group)
    exact = _integer_grads(W * S, T * M, gen)
    noisy = [(torch.randn(W * S, generator=gen) * 1e-3).bfloat16() for _ in range(T * M)]
    exact_dev = [g.cuda() for g in exact]
    noisy_dev = [g.cuda() for g in noisy]
    streams = [torch.cuda.Stream() for _ in range(T)]
    torch.cuda.synchronize()
    for minibatch in range(2):
        red.clear_accumulations()

        def body(t):
            with torch.cuda.stream(streams[t]):
                for m in range(M):
                    red.scatter_accumulate("k", exact_dev[t * M + m], group)
                    red.scatter_accumulate("r", noisy_dev[t * M + m], group)

        _run_threads(T, body)
        red.sync(group)
        want_k = [torch.zeros(S) for _ in range(W)]
        want_r = [torch.zeros(S) for _ in range(W)]
        for g in exact:
            oracle.scatter_accumulate(want_k, g)
        for g in noisy:
            oracle.scatter_accumulate(want_r, g)
        for r in range(W):
            assert_bit_equal(red.get_peer_accumulations("k")[r], want_k[r], f"minibatch {minibatch} rank {r}")
            # tolerance case: the order between streams is free; rtol 1e-6 of the sum's scale
            torch.testing.assert_close(red.get_peer_accumulations("r")[r].cpu(), want_r[r], rtol=1e-6,
                                       atol=1e-6 * 24 * 4e-3)


@pytest.mark.parametrize("lazy", [False, True])
def test_chained_streams_keep_the_callers_order_bit_for_bit(make_world, lazy):
    """One host thread issues the microbatches in order, each on the next of three streams, with
    nothing but the service ordering them: the sums are those of the sequential oracle, bit for
    bit, over two minibatches (the clear of the second runs on yet another stream)."""
    from odc_amd import ReductionService

    M = 9
    group = make_world(W, 64 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    gen = torch.Generator().manual_seed(4)
    grads = [(torch.randn(W * S, generator=gen) * 1e-3).bfloat16() for _ in range(M)]
    dev = [g.cuda() for g in grads]
    streams = [torch.cuda.Stream() for _ in range(3)]
    red.register("k", (S,), torch.bfloat16, torch.float32, group)
    torch.cuda.synchronize()
    for minibatch in range(2):
        with torch.cuda.stream(streams[(minibatch + 1) % 3]):
            red.clear_accumulations()
        for m in range(M):
            with torch.cuda.stream(streams[m % 3]):
                red.scatter_accumulate("k", dev[m], group)
        with torch.cuda.stream(streams[2]):
            published = red.publish(["k"], out_dtype=torch.bfloat16, divisor=float(W))[0]
        red.sync(group)
        want = [torch.zeros(S) for _ in range(W)]
        for g in grads:
            oracle.scatter_accumulate(want, g)
        want[0] = oracle.fsdp2_average(want[0], W)  # the publishing rank (0) divides in place
        for r in range(W):
            assert_bit_equal(red.get_peer_accumulations("k")[r], want[r], f"minibatch {minibatch} rank {r}")
        assert_bit_equal(published, want[0].bfloat16(), f"minibatch {minibatch}: published copy")


def test_multi_key_launches_from_two_streams(make_world):
    """Launches that cover several keys at once, alternating between two streams, with a
    single-key launch on a third: every key sees its adds in call order."""
    from odc_amd import ReductionService

    group = make_world(W, 96 << 20)
    red = ReductionService(accumulation_dtype=torch.float32)
    gen = torch.Generator().manual_seed(6)
    keys = ["a", "b", "c"]
    n = 800_000
    rounds = 6
    grads = [[(torch.randn(W * n, generator=gen) * 1e-3).bfloat16() for _ in keys] for _ in range(rounds)]
    dev = [[g.cuda() for g in mb] for mb in grads]
    s0, s1, s2 = (torch.cuda.Stream() for _ in range(3))
    torch.cuda.synchronize()
    for i in range(rounds):
        with torch.cuda.stream(s0 if i % 2 == 0 else s1):
            red.scatter_accumulate_multi(keys, dev[i], group)
        with torch.cuda.stream(s2):
            red.scatter_accumulate("b", dev[i][1], group)
    red.sync(group)
    want = {k: [torch.zeros(n) for _ in range(W)] for k in keys}
    for i in range(rounds):
        for k, g in zip(keys, grads[i]):
            oracle.scatter_accumulate(want[k], g)
        oracle.scatter_accumulate(want["b"], grads[i][1])
    for k in keys:
        for r in range(W):
            assert_bit_equal(red.get_peer_accumulations(k)[r], want[k][r], f"key {k} rank {r}")


def test_gather_on_another_stream_waits_for_the_conversion(make_world):
    """convert_symm_buffer on one stream, the gather that reads its output on another: the
    gather must see the converted shards (fp32 -> bf16, all W ranks in one launch)."""
    from odc_amd import GatherService, SymmBufferRegistry

    n = 3_000_001
    group = make_world(W, 64 << 20)
    registry = SymmBufferRegistry.get_instance()
    gather = GatherService()
    registry.allocate_symm_buffer("master", (n,), torch.float32)
    registry.allocate_symm_buffer("compute", (n,), torch.bfloat16)
    gen = torch.Generator().manual_seed(8)
    s_convert, s_gather = torch.cuda.Stream(), torch.cuda.Stream()
    out = torch.empty(W * n, dtype=torch.bfloat16, device="cuda")
    for step in range(3):
        shards = [torch.randn(n, generator=gen) * 0.02 for _ in range(W)]
        for peer, shard in zip(registry.peer_tensors["master"], shards):
            peer.copy_(shard)
        torch.cuda.synchronize()
        with torch.cuda.stream(s_convert):
            gather.convert_symm_buffer("compute", "master")
        with torch.cuda.stream(s_gather):
            gather.gather_into_tensor(out, registry.get_symm_buffer("compute"), group)
        torch.cuda.synchronize()
        want = torch.cat([s.bfloat16() for s in shards])
        assert_bit_equal(out, want, f"step {step}")


@pytest.mark.parametrize("lazy", [False, True])
@pytest.mark.parametrize("seed", range(4))
def test_random_schedules_over_streams_match_the_sequential_oracle(make_world, seed, lazy):
    """One host thread issues a random schedule of whole-key accumulates, multi-key accumulates,
    slice accumulates, clears and publishes, every call on a randomly chosen one of four streams
    (the default stream included). The caller's order is the only order there is, so after every
    minibatch all accumulations must equal the sequential oracle bit for bit."""
    import random

    from odc_amd import ReductionService

    rng = random.Random(1000 * seed + lazy)
    Wl, n = 4, 300_000
    group = make_world(Wl, 96 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    gen = torch.Generator().manual_seed(seed)
    keys = ["a", "b", "c", "d"]
    slices = [(0, 100_000), (100_000, 4096), (110_000, 150_000)]  # of key "s": two gaps
    total_s = 280_000
    pool = [(torch.randn(Wl * n, generator=gen) * 1e-3).bfloat16() for _ in range(6)]
    pool_dev = [g.cuda() for g in pool]
    slice_pool = [[(torch.randn(Wl * m, generator=gen) * 1e-3).bfloat16() for _, m in slices] for _ in range(3)]
    slice_dev = [[g.cuda() for g in gs] for gs in slice_pool]
    streams = [torch.cuda.default_stream()] + [torch.cuda.Stream() for _ in range(3)]
    for k in keys:
        red.register(k, (n,), torch.bfloat16, torch.float32, group)
    red.scatter_accumulate_slices("s", slice_dev[0], [o for o, _ in slices], [m for _, m in slices], group,
                                  accumulation_numel=total_s)
    torch.cuda.synchronize()
    want = {k: [torch.zeros(n) for _ in range(Wl)] for k in keys}
    want["s"] = [torch.zeros(total_s) for _ in range(Wl)]
    for minibatch in range(3):
        with torch.cuda.stream(rng.choice(streams)):
            red.clear_accumulations()
        for accs in want.values():
            for a in accs:
                a.zero_()
        for _ in range(rng.randrange(6, 14)):
            op = rng.choice(["one", "multi", "slices", "publish"])
            with torch.cuda.stream(rng.choice(streams)):
                if op == "one":
                    k, g = rng.choice(keys), rng.randrange(len(pool))
                    red.scatter_accumulate(k, pool_dev[g], group)
                    oracle.scatter_accumulate(want[k], pool[g])
                elif op == "multi":
                    ks = rng.sample(keys, rng.randrange(2, 5))
                    gs = [rng.randrange(len(pool)) for _ in ks]
                    red.scatter_accumulate_multi(ks, [pool_dev[g] for g in gs], group)
                    for k, g in zip(ks, gs):
                        oracle.scatter_accumulate(want[k], pool[g])
                elif op == "slices":
                    g = rng.randrange(len(slice_pool))
                    red.scatter_accumulate_slices("s", slice_dev[g], [o for o, _ in slices], [m for _, m in slices], group)
                    for (o, m), t in zip(slices, slice_pool[g]):
                        oracle.scatter_accumulate([w[o : o + m] for w in want["s"]], t)
                else:
                    k = rng.choice(keys)
                    red.publish([k], divisor=2.0)  # rank 0 halves its accumulation in place (exact)
                    want[k][0] /= 2.0
        red.sync(group)
        for k, accs in want.items():
            # reading settles what a lazy clear still owes a key that the minibatch never touched
            for r, acc in enumerate(red.get_peer_accumulations(k)):
                assert_bit_equal(acc, accs[r], f"seed {seed} minibatch {minibatch} key {k} rank {r}")


def _keep_busy(stream, milliseconds=60):
    """Queue a kernel that occupies ``stream`` for a while, so that whatever is queued behind it
    starts long after work issued later on other streams would, if nothing ordered them."""
    a = torch.randn(4096, 4096, device="cuda")
    with torch.cuda.stream(stream):
        start = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(int(milliseconds * 12)):  # a 4096^3 fp32 GEMM takes well over 80 us here
            a = a @ a.clamp(-1e-3, 1e-3)
    return a


@pytest.mark.parametrize("lazy", [False, True])
def test_order_is_the_callers_even_when_the_earlier_stream_is_busy(make_world, lazy):
    """Deterministic form of the ordering test: the stream of the EARLIER call is kept busy, so
    without the service's ordering the later calls (a clear, a publish that halves, another
    accumulate, on other streams) would run first and leave different values, not just a
    different rounding."""
    from odc_amd import ReductionService

    Wl, n = 4, 200_000
    group = make_world(Wl, 32 << 20)
    red = ReductionService(accumulation_dtype=torch.float32, lazy_clear=lazy)
    gen = torch.Generator().manual_seed(12)
    g1, g2, g3 = ((torch.randn(Wl * n, generator=gen) * 1e-3).bfloat16() for _ in range(3))
    d1, d2, d3 = g1.cuda(), g2.cuda(), g3.cuda()
    red.register("k", (n,), torch.bfloat16, torch.float32, group)
    s1, s2, s3 = (torch.cuda.Stream() for _ in range(3))
    torch.cuda.synchronize()

    # accumulate g1 behind a busy stream, then halve on another stream, then add g2 on a third
    red.clear_accumulations()
    busy = _keep_busy(s1)
    with torch.cuda.stream(s1):
        red.scatter_accumulate("k", d1, group)
    with torch.cuda.stream(s2):
        red.publish(["k"], divisor=2.0)
    with torch.cuda.stream(s3):
        red.scatter_accumulate("k", d2, group)
    red.sync(group)
    want = [torch.zeros(n) for _ in range(Wl)]
    oracle.scatter_accumulate(want, g1)
    want[0] /= 2.0  # the publishing rank is rank 0
    oracle.scatter_accumulate(want, g2)
    for r in range(Wl):
        assert_bit_equal(red._registry_peers("k")[r], want[r], f"accumulate, publish, accumulate: rank {r}")

    # accumulate g3 behind a busy stream, then a new minibatch (clear) and g1 on other streams
    busy = _keep_busy(s2)
    with torch.cuda.stream(s2):
        red.scatter_accumulate("k", d3, group)
    with torch.cuda.stream(s3):
        red.clear_accumulations()
    with torch.cuda.stream(s1):
        red.scatter_accumulate("k", d1, group)
    red.sync(group)
    want = [torch.zeros(n) for _ in range(Wl)]
    oracle.scatter_accumulate(want, g1)
    for r in range(Wl):
        assert_bit_equal(red.get_peer_accumulations("k")[r], want[r], f"accumulate, clear, accumulate: rank {r}")
    del busy


def test_gather_waits_for_a_conversion_on_a_busy_stream(make_world):
    """The conversion is queued behind a busy stream; gathers issued afterwards on other streams
    (several: streams that share a hardware queue with the conversion's are ordered by the queue
    itself) must still read the converted shards, not the copy made before."""
    from odc_amd import GatherService, SymmBufferRegistry

    Wl, n = 4, 100_003
    group = make_world(Wl, 16 << 20)
    registry = SymmBufferRegistry.get_instance()
    gather = GatherService()
    registry.allocate_symm_buffer("master", (n,), torch.float32)
    registry.allocate_symm_buffer("compute", (n,), torch.bfloat16)
    gen = torch.Generator().manual_seed(9)
    s_convert = torch.cuda.Stream()
    s_gathers = [torch.cuda.Stream() for _ in range(5)]
    outs = [torch.empty(Wl * n, dtype=torch.bfloat16, device="cuda") for _ in s_gathers]
    for step in range(2):
        shards = [torch.randn(n, generator=gen) * 0.02 for _ in range(Wl)]
        for peer, shard in zip(registry.peer_tensors["master"], shards):
            peer.copy_(shard)
        torch.cuda.synchronize()
        busy = _keep_busy(s_convert)
        with torch.cuda.stream(s_convert):
            gather.convert_symm_buffer("compute", "master")
        for stream, out in zip(s_gathers, outs):
            with torch.cuda.stream(stream):
                gather.gather_into_tensor(out, registry.get_symm_buffer("compute"), group)
        torch.cuda.synchronize()
        want = torch.cat([s.bfloat16() for s in shards])
        for k, out in enumerate(outs):
            assert_bit_equal(out, want, f"step {step}, gather stream {k}")
        del busy
