"""Shared helpers of the GPU parity tests."""

import torch

_INT = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def bits(t: torch.Tensor) -> torch.Tensor:
    """Integer view for bit-exact, NaN-safe comparison."""
    return t.contiguous().view(_INT[t.element_size()])


def assert_bit_equal(got: torch.Tensor, want: torch.Tensor, what=""):
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, f"{what}: {got.shape} {got.dtype} vs {want.shape} {want.dtype}"
    if not torch.equal(bits(got), bits(want)):
        bad = (bits(got) != bits(want)).flatten().nonzero().flatten()
        i = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.numel()} of {got.numel()} elements differ; first at {i}: "
            f"got {got.flatten()[i].item()!r} want {want.flatten()[i].item()!r}"
        )


def put_shards(registry, key, shards):
    """Each virtual rank publishes its shard, as each process does in the reference
    (examples/all_gather.py:82-84). Returns rank 0's symmetric tensor."""
    from odc_amd import virtual_rank

    for r, s in enumerate(shards):
        with virtual_rank(r):
            registry.update_symm_buffer(key, s.cuda())
    return registry.peer_tensors[key][0]


def device_randn_bf16(n, gen, scale):
    return (torch.randn(n, generator=gen, device="cuda") * scale).bfloat16()
