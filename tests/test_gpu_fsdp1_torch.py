"""torch's FullyShardedDataParallel (FSDP1) trained through the primitives: one process plays rank 0
of a W-rank group over torch's "fake" process-group backend; all W flat-parameter shards live in the
symmetric arena. Checked against the same model run unsharded, with the oracle doing the
accumulation arithmetic."""

import copy
import math

import pytest
import torch
import torch.distributed as dist

from helpers import assert_bit_equal
from oracle import odc_oracle as oracle
from test_gpu_fsdp2_torch import Block, Toy

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["eager", "lazy"], autouse=True)
def clear_mode(request, monkeypatch):
    """Every test here runs with the reference's eager clears (the default) and with lazy clears
    (ODC_LAZY_CLEAR=1, read when the FSDP patches build their ReductionService)."""
    monkeypatch.setenv("ODC_LAZY_CLEAR", "1" if request.param == "lazy" else "0")
    return request.param


@pytest.fixture
def fake_process_group():
    from torch.testing._internal.distributed.fake_pg import FakeStore

    def _init(world_size):
        dist.init_process_group("fake", rank=0, world_size=world_size, store=FakeStore())

    yield _init
    from odc_amd.fsdp import fsdp1

    fsdp1.unpatch_fsdp1()
    if dist.is_initialized():
        dist.destroy_process_group()


@pytest.mark.parametrize("shard_copies", [False, True], ids=["converting gather", "compute-dtype shards"])
@pytest.mark.parametrize("W", [4, 8])
def test_fsdp1_minibatch_through_the_primitives(make_world, fake_process_group, W, shard_copies):
    """``compute-dtype shards``: the gathers read a bf16 copy of the fp32 shards that is converted
    once per minibatch; the forward after the optimizer step must see the updated shards, with
    and without a hook in between."""
    from torch.distributed.fsdp import FullyShardedDataParallel as FSDP
    from torch.distributed.fsdp import MixedPrecision
    from torch.distributed.fsdp._common_utils import clean_tensor_name
    from torch.distributed.fsdp.wrap import ModuleWrapPolicy

    from odc_amd import SymmBufferRegistry
    from odc_amd.fsdp import fsdp1

    fake_process_group(W)
    group = make_world(W, 64 << 20)
    # bf16 gradients into fp32 accumulations
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32, compute_dtype_shards=shard_copies)
    conversions = []
    convert = fsdp1.get_gather_service().convert_symm_buffer
    fsdp1.get_gather_service().convert_symm_buffer = lambda *a, **k: (conversions.append(a), convert(*a, **k))[1]

    torch.manual_seed(0)
    model = Toy().cuda()
    reference = copy.deepcopy(model)
    full_params = {name: p.detach().clone() for name, p in reference.named_parameters()}
    fsdp_model = FSDP(
        model,
        auto_wrap_policy=ModuleWrapPolicy({Block}),
        mixed_precision=MixedPrecision(param_dtype=torch.bfloat16),
        device_id=torch.cuda.current_device(),
        use_orig_params=False,
    )
    units = []  # (handle, [full parameter names in flat order])
    for name, module in fsdp_model.named_modules():
        if isinstance(module, FSDP) and module._handle is not None:
            prefix = clean_tensor_name(name)
            fqns = [f"{prefix}.{f}" if prefix else f for f in module._handle.flat_param._fqns]
            units.append((module._handle, fqns))
    assert len(units) == 4
    registry = SymmBufferRegistry.get_instance()
    for handle, fqns in units:
        flat = torch.cat([full_params[f].reshape(-1) for f in fqns])
        peers = registry.get_peer_tensors(handle.flat_param.data)
        for r in range(W):  # every virtual rank's shard was published when the unit was wrapped
            assert_bit_equal(peers[r], oracle.fsdp1_get_shard(flat, r, W), f"shard {r} of {fqns[0]}...")

    ref_compute = copy.deepcopy(reference).bfloat16()
    g = torch.Generator().manual_seed(1)
    batches = [torch.randn(16, 32, generator=g).cuda() for _ in range(3)]
    pre = fsdp_model._gradient_predivide_factor
    post = fsdp_model._gradient_postdivide_factor
    assert pre * post == W

    fsdp1.pre_minibatch_start(fsdp_model)
    want = [[torch.zeros(h.flat_param.numel()) for _ in range(W)] for h, _ in units]
    for x in batches:
        fsdp_model(x).float().pow(2).mean().backward()
        assert all(h.flat_param.grad is None for h, _ in units)  # published only at the optimizer step
        ref_compute.zero_grad(set_to_none=True)
        ref_compute(x.bfloat16()).float().pow(2).mean().backward()
        grads = {n: p.grad.detach().cpu() for n, p in ref_compute.named_parameters()}
        for accs, (_, fqns) in zip(want, units):
            flat_grad = torch.cat([grads[f].reshape(-1) for f in fqns])
            if pre > 1:
                flat_grad.div_(pre)  # in bf16, as torch does before the reduce-scatter
            oracle.scatter_accumulate(accs, oracle.fsdp1_pad_grad(flat_grad, W))
    fsdp1.pre_optimizer_step(fsdp_model)
    for accs, (handle, fqns) in zip(want, units):
        expect = oracle.fsdp1_publish(accs[0].clone(), post, torch.float32)
        assert handle.flat_param.grad.dtype == torch.float32
        assert_bit_equal(handle.flat_param.grad, expect, f"flat gradient of {fqns[0]}...")

    opt = torch.optim.SGD(fsdp_model.parameters(), lr=0.1)
    opt.step()
    opt.zero_grad()
    fsdp1.pre_minibatch_start(fsdp_model)
    out = fsdp_model(batches[0])
    with torch.no_grad():  # reference: chunk 0 of every flat parameter updated, the rest unchanged
        named = dict(reference.named_parameters())
        for handle, fqns in units:
            flat = torch.cat([named[f].reshape(-1) for f in fqns])
            S = math.ceil(flat.numel() / W)
            flat[:S] = handle.flat_param.data[: min(S, flat.numel())]
            off = 0
            for f in fqns:
                named[f].copy_(flat[off : off + named[f].numel()].view_as(named[f]))
                off += named[f].numel()
    want_out = copy.deepcopy(reference).bfloat16()(batches[0].bfloat16())
    assert_bit_equal(out, want_out, "forward after the optimizer step")
    # one conversion per unit and minibatch, however many gathers
    assert len(conversions) == (2 * len(units) if shard_copies else 0)
    if shard_copies:
        # an in-place update with no hook in between: the flat parameters' version counters tell
        out.float().pow(2).mean().backward()  # leaves every unit resharded, the root's too
        with torch.no_grad():
            for handle, fqns in units:
                handle.flat_param.mul_(0.5)
                flat = torch.cat([named[f].reshape(-1) for f in fqns])
                S = math.ceil(flat.numel() / W)
                flat[:S] = handle.flat_param.data[: min(S, flat.numel())]
                off = 0
                for f in fqns:
                    named[f].copy_(flat[off : off + named[f].numel()].view_as(named[f]))
                    off += named[f].numel()
        out = fsdp_model(batches[1])
        want_out = copy.deepcopy(reference).bfloat16()(batches[1].bfloat16())
        assert_bit_equal(out, want_out, "forward after an in-place update without a hook")
        assert len(conversions) == 3 * len(units)


@pytest.mark.parametrize("extra", [
    ["--world-size", "12", "--layers", "3", "--forward-prefetch"],
    ["--world-size", "5", "--layers", "2", "--no-backward-prefetch", "--microbatches", "3"],
    ["--world-size", "12", "--layers", "3", "--shard-grad-op"],
    ["--world-size", "8", "--layers", "2", "--microbatches", "4", "--sync-every", "2"],
    ["--world-size", "12", "--layers", "3", "--forward-prefetch", "ENV:ODC_FSDP1_COMPUTE_DTYPE_SHARDS=1"],
])
def test_transformer_example_trains_bit_exactly(extra):
    """examples/fsdp1_toy.py: a small transformer under FSDP1 with forward / backward prefetching
    on and off, at uneven world sizes; every step's flat gradient shards equal the unsharded model's."""
    import subprocess
    import sys
    from pathlib import Path

    script = Path(__file__).resolve().parent.parent / "examples" / "fsdp1_toy.py"
    import os

    env = dict(os.environ)
    env.update(e[4:].split("=", 1) for e in extra if e.startswith("ENV:"))
    args = [e for e in extra if not e.startswith("ENV:")]
    proc = subprocess.run([sys.executable, str(script), "--steps", "3", *args],
                          capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert proc.stdout.count("match the unsharded model bit for bit") == 3


def test_fsdp1_with_a_frozen_unit(make_world, fake_process_group):
    """A wrapped block none of whose parameters require a gradient never reaches the
    scatter-accumulate: ``pre_optimizer_step`` leaves its gradient ``None`` and publishes the
    other units exactly."""
    from torch.distributed.fsdp import FullyShardedDataParallel as FSDP
    from torch.distributed.fsdp import MixedPrecision
    from torch.distributed.fsdp._common_utils import clean_tensor_name
    from torch.distributed.fsdp.wrap import ModuleWrapPolicy

    from odc_amd.fsdp import fsdp1

    W = 4
    fake_process_group(W)
    make_world(W, 64 << 20)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    torch.manual_seed(0)
    model = Toy().cuda()
    for p in model.layers[1].parameters():
        p.requires_grad_(False)
    reference = copy.deepcopy(model).bfloat16()
    fsdp_model = FSDP(model, auto_wrap_policy=ModuleWrapPolicy({Block}),
                      mixed_precision=MixedPrecision(param_dtype=torch.bfloat16),
                      device_id=torch.cuda.current_device(), use_orig_params=False)
    units = []
    for name, module in fsdp_model.named_modules():
        if isinstance(module, FSDP) and module._handle is not None:
            prefix = clean_tensor_name(name)
            units.append((module._handle, [f"{prefix}.{f}" if prefix else f for f in module._handle.flat_param._fqns]))
    pre, post = fsdp_model._gradient_predivide_factor, fsdp_model._gradient_postdivide_factor
    g = torch.Generator().manual_seed(2)
    batches = [torch.randn(16, 32, generator=g).cuda() for _ in range(2)]
    fsdp1.pre_minibatch_start(fsdp_model)
    want = {}
    for x in batches:
        fsdp_model(x).float().pow(2).mean().backward()
        reference.zero_grad(set_to_none=True)
        reference(x.bfloat16()).float().pow(2).mean().backward()
        grads = {n: p.grad for n, p in reference.named_parameters()}
        for u, (_, fqns) in enumerate(units):
            if grads[fqns[0]] is None:
                continue
            flat_grad = torch.cat([grads[f].detach().cpu().reshape(-1) for f in fqns])
            if pre > 1:
                flat_grad.div_(pre)
            accs = want.setdefault(u, [torch.zeros(math.ceil(flat_grad.numel() / W)) for _ in range(W)])
            oracle.scatter_accumulate(accs, oracle.fsdp1_pad_grad(flat_grad, W))
    fsdp1.pre_optimizer_step(fsdp_model)
    frozen = [u for u, (_, fqns) in enumerate(units) if fqns[0].startswith("layers.1.")]
    assert len(frozen) == 1 and frozen[0] not in want
    for u, (handle, fqns) in enumerate(units):
        if u in frozen:
            assert handle.flat_param.grad is None
        else:
            expect = oracle.fsdp1_publish(want[u][0].clone(), post, torch.float32)
            assert_bit_equal(handle.flat_param.grad, expect, f"flat gradient of {fqns[0]}...")
