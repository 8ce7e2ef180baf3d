"""The benchmark configurations at their full sizes (2-4) against the CPU oracle.

Inputs are drawn on the device from a seeded generator and mirrored to the host, so the HIP path
and the oracle see identical bits; the oracle handles these sizes in seconds."""

import pytest
import torch

from helpers import assert_bit_equal, device_randn_bf16
from odc_amd.workloads import llama3_8b_layer_shapes, numel, shard_numel, uneven_flat_numels
from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu


def _services():
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry

    return GatherService(), ReductionService(accumulation_dtype=torch.float32), SymmBufferRegistry.get_instance()


def _run_layer(make_world, W, layout, microbatches):
    shapes = llama3_8b_layer_shapes()
    numels = [numel(s) for _, s in shapes]
    if layout == "flat":
        numels = [sum(numels)]
    N = sum(numels)
    assert N == 218_112_000
    per_rank = sum((n // W) * 6 + 512 for n in numels) + (1 << 20)
    group = make_world(W, per_rank)
    gather, reduction, registry = _services()
    gen = torch.Generator(device="cuda").manual_seed(0)
    params = [device_randn_bf16(n, gen, 0.02) for n in numels]
    keys = list(range(len(numels)))
    from odc_amd import virtual_rank

    for key, p in zip(keys, params):
        for r in range(W):
            with virtual_rank(r):
                registry.update_symm_buffer(key, p.view(W, -1)[r])
    outs = [torch.full_like(p, float("nan")) for p in params]
    gather.gather_into_tensors(outs, [registry.get_symm_buffer(k) for k in keys], group)
    for o, p in zip(outs, params):  # gather of equal shards of p is p itself
        assert torch.equal(o.view(torch.int16), p.view(torch.int16))
        host = p.cpu()
        assert_bit_equal(o, oracle.gather(list(host.view(W, -1))), "gather vs oracle")
    del outs

    want = [[torch.zeros(n // W) for _ in range(W)] for n in numels]
    for _ in range(microbatches):
        grads = [device_randn_bf16(n, gen, 1e-3) for n in numels]
        reduction.scatter_accumulate_multi(keys, grads, group)
        for accs, g in zip(want, grads):
            oracle.scatter_accumulate(accs, g.cpu())
    reduction.sync(group)
    for key, accs in zip(keys, want):
        for r, acc in enumerate(reduction.get_peer_accumulations(key)):
            assert_bit_equal(acc, accs[r], f"W={W} {layout} key {key} rank {r}")


@pytest.mark.parametrize("layout", ["per-param", "flat"])
def test_config2_llama_layer_w8(make_world, layout):
    """Llama-3-8B decoder layer, W=8, a minibatch of 8 microbatches: 9 per-parameter shards in one
    multi-tensor launch, and the same 218 112 000 elements as one flat shard of 27 264 000."""
    _run_layer(make_world, 8, layout, microbatches=8)


@pytest.mark.parametrize("layout", ["per-param", "flat"])
def test_config4_small_chunks_w64(make_world, layout):
    """The same layer at W=64, a minibatch of 16 microbatches: shards from 917 504 elements down to
    the 64-element (128 B) slices of the two norm vectors."""
    _run_layer(make_world, 64, layout, microbatches=16)


def test_config3_uneven_padded_w12(make_world):
    """40 flat parameters with numel not divisible by W=12; shard = ceil(numel/12), the last
    rank's tail zero padded (FSDP1 rule); all 40 gathered by ONE fused launch; gradients are
    passed unpadded and the kernel supplies the +0 tail."""
    W, M = 12, 4
    numels = uneven_flat_numels(40, W)
    assert len(numels) == 40 and all(n % W for n in numels)
    shard = [shard_numel(n, W) for n in numels]
    per_rank = sum(s * 6 + 512 for s in shard) + (1 << 20)
    group = make_world(W, per_rank)
    gather, reduction, registry = _services()
    gen = torch.Generator(device="cuda").manual_seed(0)
    from odc_amd import virtual_rank

    host_params, locals_ = [], []
    for i, n in enumerate(numels):
        p = device_randn_bf16(n, gen, 0.02).cpu()
        host_params.append(p)
        for r in range(W):
            with virtual_rank(r):
                registry.update_symm_buffer(i, oracle.fsdp1_get_shard(p, r, W).cuda())
        locals_.append(registry.get_symm_buffer(i))
    outs = [torch.full((W * s,), float("nan"), dtype=torch.bfloat16, device="cuda") for s in shard]
    gather.gather_into_tensors(outs, locals_, group)  # 40 items, one launch
    for i, (o, p) in enumerate(zip(outs, host_params)):
        want = oracle.gather([oracle.fsdp1_get_shard(p, r, W) for r in range(W)])
        assert_bit_equal(o, want, f"param {i} (numel {numels[i]})")
        assert_bit_equal(o[: numels[i]], p, f"param {i} unpadded prefix")
        assert not o[numels[i] :].cpu().float().abs().any(), "padding must be zero"
    del outs

    keys = list(range(len(numels)))
    for k, s in zip(keys, shard):
        reduction.register(k, (s,), torch.bfloat16, torch.float32, group)
    want = [[torch.zeros(s) for _ in range(W)] for s in shard]
    for _ in range(M):
        grads = [device_randn_bf16(n, gen, 1e-3) for n in numels]
        reduction.scatter_accumulate_multi(keys, grads, group, valid_numels=numels)
        for accs, g in zip(want, grads):
            oracle.scatter_accumulate(accs, oracle.fsdp1_pad_grad(g.cpu(), W))
    reduction.sync(group)
    for k, accs in zip(keys, want):
        for r, acc in enumerate(reduction.get_peer_accumulations(k)):
            assert_bit_equal(acc, accs[r], f"param {k} rank {r}")


def test_config5_full_llama3_8b_sweep(make_world):
    """Full Llama-3-8B (34 FSDP units: embedding, 32 layers, final norm + untied lm_head; 8.03 G
    bf16 parameters, W=8, ~48 GB arena). Per microbatch: gather unit by unit in forward order, then
    scatter-accumulate unit by unit in reverse order. Values come from per-(unit, microbatch) seeded
    device generators, so they can be drawn again for checking:
      * every unit: gathered parameters equal the regenerated parameters; accumulations equal
        ((0 + g0) + g1) + ... over the 8 microbatches, computed with torch's fp32 add on the device
        (an independent implementation);
      * sampled units (embedding, two layers, head): bit-exact against the CPU oracle."""
    from odc_amd import virtual_rank
    from odc_amd.workloads import llama3_8b_units

    W, M = 8, 8
    units = llama3_8b_units()
    total = sum(numel(s) for _, unit in units for _, s in unit)
    assert total == 8_030_261_248
    per_rank = sum((numel(s) // W) * 6 + 512 for _, unit in units for _, s in unit) + (1 << 20)
    group = make_world(W, per_rank)
    gather, reduction, registry = _services()

    def draw(u, p, m, n, scale):
        gen = torch.Generator(device="cuda").manual_seed(1_000_003 * u + 1009 * p + m)
        return device_randn_bf16(n, gen, scale)

    keys = []
    for u, (_, unit) in enumerate(units):
        ks = []
        for p, (_, shape) in enumerate(unit):
            n = numel(shape)
            full = draw(u, p, -1, n, 0.02)
            for r in range(W):
                with virtual_rank(r):
                    registry.update_symm_buffer((u, p), full.view(W, -1)[r])
            reduction.register((u, p), (n // W,), torch.bfloat16, torch.float32, group)
            ks.append((u, p))
        keys.append(ks)
    sampled = {0, 1, 17, len(units) - 1}
    outs_by_shape = {}
    for m in range(M):
        for u, (_, unit) in enumerate(units):  # forward: gather
            sig = tuple(numel(s) for _, s in unit)
            if sig not in outs_by_shape:
                outs_by_shape[sig] = [torch.empty(n, dtype=torch.bfloat16, device="cuda") for n in sig]
            outs = outs_by_shape[sig]
            gather.gather_into_tensors(outs, [registry.get_symm_buffer(k) for k in keys[u]], group)
            if m == 0:
                for p, o in enumerate(outs):
                    assert torch.equal(o.view(torch.int16), draw(u, p, -1, o.numel(), 0.02).view(torch.int16)), (u, p)
        for u in reversed(range(len(units))):  # backward: scatter-accumulate
            grads = [draw(u, p, m, numel(s), 1e-3) for p, (_, s) in enumerate(units[u][1])]
            reduction.scatter_accumulate_multi(keys[u], grads, group)
    reduction.sync(group)
    for u, (_, unit) in enumerate(units):
        for p, (_, shape) in enumerate(unit):
            n = numel(shape)
            expect = torch.zeros(n, device="cuda")
            accs = [torch.zeros(n // W) for _ in range(W)] if u in sampled else None
            for m in range(M):
                g = draw(u, p, m, n, 1e-3)
                expect += g.float()
                if accs is not None:
                    oracle.scatter_accumulate(accs, g.cpu())
                del g
            got = torch.cat(list(reduction.get_peer_accumulations((u, p))))
            assert torch.equal(got.view(torch.int32), expect.view(torch.int32)), (u, p)
            if accs is not None:
                assert_bit_equal(got, torch.cat(accs), f"unit {u} param {p} vs oracle")
            del expect, got


@pytest.mark.parametrize("W", [8, 12])
def test_layer_with_fp32_master_shards_cast_gather_and_publish(make_world, W):
    """The layer at full size the way FSDP mixed precision runs it: fp32 master shards gathered
    as bf16 in one pass (against torch's own CPU ``.to(bfloat16)`` of the concatenation), bf16
    gradients into fp32 accumulations, then the end-of-minibatch divide by W and bf16 copy
    (against the oracle's torch CPU division and cast). W=12 divides with a true division."""
    from odc_amd import virtual_rank

    shapes = llama3_8b_layer_shapes()
    numels = [numel(s) for _, s in shapes]
    S = [shard_numel(n, W) for n in numels]
    group = make_world(W, sum(s * 8 + 512 for s in S) + (1 << 20))
    gather, reduction, registry = _services()
    gen = torch.Generator(device="cuda").manual_seed(4)
    keys = list(range(len(numels)))
    shards = []
    for key, s in zip(keys, S):
        registry.allocate_symm_buffer(key, (s,), torch.float32)
        for peer in registry.peer_tensors[key]:
            peer.normal_(0.0, 0.02, generator=gen)
        shards.append([p.cpu() for p in registry.peer_tensors[key]])
    outs = [torch.empty(W * s, dtype=torch.bfloat16, device="cuda") for s in S]
    with virtual_rank(W - 1):
        gather.gather_into_tensors(outs, [registry.get_symm_buffer(k) for k in keys], group)
    for o, sh in zip(outs, shards):
        assert_bit_equal(o, torch.cat(sh).to(torch.bfloat16), "converting gather")
    del outs

    want = [[torch.zeros(s) for _ in range(W)] for s in S]
    for _ in range(2):
        grads = [device_randn_bf16(W * s, gen, 1e-3) for s in S]
        reduction.scatter_accumulate_multi(keys, grads, group)
        for accs, g in zip(want, grads):
            oracle.scatter_accumulate(accs, g.cpu())
    reduction.sync(group)
    for rank in (0, W - 1):
        with virtual_rank(rank):
            published = reduction.publish(keys, out_dtype=torch.bfloat16, divisor=float(W))
            for key, out, accs in zip(keys, published, want):
                averaged = oracle.fsdp2_average(accs[rank].clone(), W)
                assert_bit_equal(reduction.get_accumulation(key), averaged, f"rank {rank} key {key}: acc / W")
                assert_bit_equal(out, averaged.to(torch.bfloat16), f"rank {rank} key {key}: bf16 copy")
