"""The committed vectors of tests/golden/vectors.npz: the oracle must reproduce them here (so it
cannot drift unnoticed), and the HIP path must reproduce them on the GPU."""

from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import odc_oracle as oracle

VEC = Path(__file__).resolve().parent / "golden" / "vectors.npz"

ACC_CASES = [("bf16_f32", torch.bfloat16, torch.float32), ("f16_f32", torch.float16, torch.float32),
             ("bf16_bf16", torch.bfloat16, torch.bfloat16)]


@pytest.fixture(scope="module")
def vec():
    return np.load(VEC, allow_pickle=False)


def t(arr, dtype):
    return torch.from_numpy(np.ascontiguousarray(arr)).view(dtype)


def same_bits(tensor, arr):
    got = tensor.detach().cpu().contiguous()
    got = got.view({2: torch.int16, 4: torch.int32}[got.element_size()]).numpy()
    return np.array_equal(got, arr)


def test_vectors_are_meaningful(vec):
    for tag, gdt, adt in ACC_CASES:
        out = t(vec[f"acc_{tag}_out"], adt).float()
        assert torch.isfinite(out).all() and (out != 0).float().mean() > 0.99
    assert not np.array_equal(vec["cast_out"].astype(np.int32) << 16, vec["cast_shards"].reshape(-1))  # rounding happened


def test_oracle_reproduces_the_vectors(vec):
    shards = [torch.from_numpy(s) for s in vec["gather_shards"]]
    assert np.array_equal(oracle.gather(shards).numpy(), vec["gather_out"])
    for tag, gdt, adt in ACC_CASES:
        grads = vec[f"acc_{tag}_grads"]
        W, S = vec[f"acc_{tag}_out"].shape
        accs = [torch.zeros(S, dtype=adt) for _ in range(W)]
        for g in grads:
            oracle.scatter_accumulate(accs, t(g, gdt))
        for r in range(W):
            assert same_bits(accs[r], vec[f"acc_{tag}_out"][r]), (tag, r)
    flat = t(vec["fsdp1_flat"], torch.bfloat16)
    W = vec["fsdp1_shards"].shape[0]
    for r in range(W):
        assert same_bits(oracle.fsdp1_get_shard(flat, r, W), vec["fsdp1_shards"][r])
    accs = [torch.zeros(vec["fsdp1_acc"].shape[1]) for _ in range(W)]
    oracle.scatter_accumulate(accs, oracle.fsdp1_pad_grad(t(vec["fsdp1_grad"], torch.bfloat16), W))
    for r in range(W):
        assert same_bits(accs[r], vec["fsdp1_acc"][r])
    assert same_bits(oracle.fsdp1_publish(accs[1].clone(), 4.0, torch.bfloat16), vec["fsdp1_published_div4_bf16"])
    assert same_bits(oracle.fsdp2_average(accs[2].clone(), 12), vec["fsdp2_averaged_div12"])
    f32 = [t(s, torch.float32) for s in vec["cast_shards"]]
    assert same_bits(oracle.gather_cast(f32, torch.bfloat16), vec["cast_out"])


@pytest.mark.gpu
def test_hip_path_reproduces_the_vectors(vec, make_world):
    from odc_amd import GatherService, ReductionService, SymmBufferRegistry, virtual_rank
    from odc_amd.fsdp import fsdp1

    # gather (W=3)
    group = make_world(3, 1 << 20)
    registry, gather = SymmBufferRegistry.get_instance(), GatherService()
    for r, s in enumerate(vec["gather_shards"]):
        with virtual_rank(r):
            registry.update_symm_buffer("g", torch.from_numpy(s).cuda())
    out = torch.empty(vec["gather_out"].shape, dtype=torch.int16, device="cuda")
    gather.gather_into_tensor(out, registry.get_symm_buffer("g"), group)
    assert np.array_equal(out.cpu().numpy(), vec["gather_out"])
    torch.cuda.synchronize()
    registry.finalize()
    from odc_amd.primitives import utils

    utils.finalize_distributed()

    # scatter-accumulate, FSDP1 padding and publish, gather with cast (W=4)
    group = make_world(4, 1 << 20)
    registry, gather = SymmBufferRegistry.get_instance(), GatherService()
    for tag, gdt, adt in ACC_CASES:
        red = ReductionService(accumulation_dtype=adt)
        for g in vec[f"acc_{tag}_grads"]:
            red.scatter_accumulate(tag, t(g, gdt).cuda(), group)
        red.sync(group)
        for r, acc in enumerate(red.get_peer_accumulations(tag)):
            assert same_bits(acc, vec[f"acc_{tag}_out"][r]), (tag, r)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    flat = torch.nn.Parameter(t(vec["fsdp1_flat"], torch.bfloat16).cuda(), requires_grad=False)
    for r in range(4):
        shard, _ = fsdp1.get_shard(flat, r, 4)
        assert same_bits(shard, vec["fsdp1_shards"][r])
    fsdp1.reduce_grad(flat, t(vec["fsdp1_grad"], torch.bfloat16).cuda(), group)
    service = fsdp1.get_reduction_service()
    service.sync(group)
    for r, acc in enumerate(service.get_peer_accumulations(id(flat))):
        assert same_bits(acc, vec["fsdp1_acc"][r])
    with virtual_rank(1):
        (published,) = service.publish([id(flat)], out_dtype=torch.bfloat16, divisor=4.0)
        service.sync(group)
        assert same_bits(published, vec["fsdp1_published_div4_bf16"])
    with virtual_rank(2):
        service.publish([id(flat)], divisor=12.0)  # in place, a true division
        service.sync(group)
        assert same_bits(service.get_accumulation(id(flat)), vec["fsdp2_averaged_div12"])
    for r, s in enumerate(vec["cast_shards"]):
        with virtual_rank(r):
            registry.update_symm_buffer("c", t(s, torch.float32).cuda())
    out = torch.empty(vec["cast_out"].shape, dtype=torch.bfloat16, device="cuda")
    gather.gather_into_tensor(out, registry.get_symm_buffer("c"), group)
    assert same_bits(out, vec["cast_out"])
