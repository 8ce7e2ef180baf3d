"""Sizes past 2^32 bytes and 2^31 elements in ONE item: 64-bit offsets and indices everywhere.
Too large for the CPU oracle to finish in seconds, so the checks are the size-independent
properties: block r of a gather bit-equals shard r; an accumulation after two calls bit-equals
``(+0 + g) + g`` computed by torch's own device add (one IEEE fp32 add per element, exact
widening); bytes beyond the ends stay untouched."""

import pytest
import torch

from helpers import bits

pytestmark = pytest.mark.gpu


def test_gather_past_four_gib(make_world):
    from odc_amd import GatherService, SymmBufferRegistry

    W, S = 8, (640 << 20) + 3  # odd shard bytes: blocks of the output start at odd addresses
    group = make_world(W, S + (1 << 20))
    registry = SymmBufferRegistry.get_instance()
    registry.allocate_symm_buffer("big", (S,), torch.uint8)
    gen = torch.Generator(device="cuda").manual_seed(1)
    for peer in registry.peer_tensors["big"]:
        peer.view(torch.uint8)[: S - 3].view(torch.int64).random_(generator=gen)
        peer[S - 3 :] = 0x5A
    pad = 256
    buf = torch.full((W * S + 2 * pad,), 0xEE, dtype=torch.uint8, device="cuda")
    assert W * S > (1 << 32)
    out = buf[pad : pad + W * S]
    GatherService().gather_into_tensor(out, registry.get_symm_buffer("big"), group)
    torch.cuda.synchronize()
    for r, peer in enumerate(registry.peer_tensors["big"]):
        assert torch.equal(out[r * S : (r + 1) * S], peer), f"block {r}"
    assert (buf[:pad] == 0xEE).all() and (buf[pad + W * S :] == 0xEE).all()


def test_scatter_accumulate_past_two_gi_elements(make_world):
    from odc_amd import ReductionService

    W, S = 8, (300 << 20) + 1
    n = W * S
    assert n > (1 << 31)
    group = make_world(W, 4 * S + (1 << 20))
    red = ReductionService(accumulation_dtype=torch.float32)
    gen = torch.Generator(device="cuda").manual_seed(2)
    grad = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    step = 1 << 28
    for lo in range(0, n, step):  # generated in pieces to bound the fp32 temporaries
        hi = min(n, lo + step)
        grad[lo:hi] = torch.randn(hi - lo, generator=gen, device="cuda") * 1e-3
    red.scatter_accumulate("big", grad, group)   # store form: acc = +0 + g
    red.scatter_accumulate("big", grad, group)   # read-modify-write
    red.sync(group)
    for r, acc in enumerate(red.get_peer_accumulations("big")):
        g = grad[r * S : (r + 1) * S].float()
        want = torch.zeros(S, device="cuda").add_(g).add_(g)
        assert torch.equal(bits(acc), bits(want)), f"rank {r}"
        del g, want
    # the padded form at the same size: the last 5 elements of the gradient do not exist
    red.clear_accumulations()
    red.scatter_accumulate_multi(["big"], [grad[: n - 5]], group, valid_numels=[n - 5])
    last = red.get_peer_accumulations("big")[W - 1]
    assert torch.equal(bits(last[: S - 5]), bits(torch.zeros(S - 5, device="cuda").add_(grad[(W - 1) * S : n - 5].float())))
    assert torch.equal(bits(last[S - 5 :]), torch.zeros(5, dtype=torch.int32, device="cuda"))


def test_far_end_of_a_128_gib_arena(make_world):
    """Rank regions of 16 GiB each (the reference's launch script reserves 30 GB per rank):
    buffers parked at the far end of every region, byte offsets past 2^33 and rank strides past
    2^34, through gather and both forms of scatter-accumulate."""
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry
    from odc_amd.primitives import utils

    W, per_rank, n = 8, 16 << 30, 1 << 20
    group = make_world(W, per_rank)
    arena = utils.get_world().arena
    arena.alloc(per_rank - (1 << 30))  # everything after this lands in the last GiB of a region
    registry = SymmBufferRegistry.get_instance()
    registry.allocate_symm_buffer("far", (n,), torch.float32)
    assert registry.get_offset("far") >= per_rank - (1 << 30)
    for r, peer in enumerate(registry.peer_tensors["far"]):
        peer.fill_(float(r))
    out = torch.empty(W * n, device="cuda")
    GatherService().gather_into_tensor(out, registry.get_symm_buffer("far"), group)
    assert torch.equal(out.view(W, n), torch.arange(W, dtype=torch.float32, device="cuda")[:, None].expand(W, n))
    red = ReductionService(accumulation_dtype=torch.float32)
    grad = torch.arange(W * n, device="cuda").remainder(251).bfloat16()
    red.scatter_accumulate("k", grad, group)
    red.scatter_accumulate("k", grad, group)
    red.sync(group)
    for r, acc in enumerate(red.get_peer_accumulations("k")):
        assert torch.equal(acc, grad[r * n : (r + 1) * n].float() * 2), f"rank {r}"
