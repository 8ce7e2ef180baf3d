"""torch's own fully_shard (FSDP2) trained through the primitives: one process plays rank 0 of a
W-rank mesh over torch's "fake" process-group backend; the other ranks' shards are passive memory
in the symmetric arena. Checked against the same model run unsharded."""

import copy
import math

import pytest
import torch
import torch.distributed as dist
import torch.nn as nn

from helpers import assert_bit_equal
from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["eager", "lazy"], autouse=True)
def clear_mode(request, monkeypatch):
    """Every test here runs with the reference's eager clears (the default) and with lazy clears
    (ODC_LAZY_CLEAR=1, read when the FSDP patches build their ReductionService)."""
    monkeypatch.setenv("ODC_LAZY_CLEAR", "1" if request.param == "lazy" else "0")
    return request.param


class Block(nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.norm = nn.LayerNorm(dim)
        self.up = nn.Linear(dim, hidden)
        self.down = nn.Linear(hidden, dim, bias=False)

    def forward(self, x):
        return x + self.down(torch.relu(self.up(self.norm(x))))


class Toy(nn.Module):
    def __init__(self, dim=96, hidden=50, layers=3, out=10):
        super().__init__()
        self.inp = nn.Linear(32, dim)
        self.layers = nn.ModuleList([Block(dim, hidden) for _ in range(layers)])
        self.head = nn.Linear(dim, out)

    def forward(self, x):
        x = self.inp(x)
        for layer in self.layers:
            x = layer(x)
        return self.head(x)


@pytest.fixture
def fake_process_group():
    from torch.testing._internal.distributed.fake_pg import FakeStore

    def _init(world_size):
        dist.init_process_group("fake", rank=0, world_size=world_size, store=FakeStore())

    yield _init
    from odc_amd.fsdp import fsdp2

    fsdp2.unpatch_fsdp2()
    if dist.is_initialized():
        dist.destroy_process_group()


@pytest.mark.parametrize("dims", [(96, 50), (192, 1100)], ids=["small", "wide"])
@pytest.mark.parametrize("W", [4, 8])
@pytest.mark.parametrize("mixed", [True, False, "compute-dtype shards"])
def test_fully_shard_minibatch_through_the_primitives(make_world, fake_process_group, W, mixed, dims):
    """`wide`: the weight shards exceed one tile (4096 elements), so the groups' accumulations
    have their slices on tile boundaries, with gaps after the small ones (norms, biases).
    `compute-dtype shards`: mixed precision with the gathers reading a bf16 copy of the shards
    that is converted once per minibatch; the forward after the optimizer step must see the
    updated shards."""
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.fsdp import MixedPrecisionPolicy, fully_shard

    from odc_amd.fsdp import fsdp2

    fake_process_group(W)
    mesh = init_device_mesh("cuda", (W,))
    make_world(W, 64 << 20)
    fsdp2.patch_fsdp2(compute_dtype_shards=mixed == "compute-dtype shards")

    torch.manual_seed(0)
    model = Toy(dim=dims[0], hidden=dims[1]).cuda()
    reference = copy.deepcopy(model)
    full_params = {name: p.detach().clone() for name, p in reference.named_parameters()}
    kwargs = {"mesh": mesh}
    if mixed:
        kwargs["mp_policy"] = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32)
    for layer in model.layers:
        fully_shard(layer, **kwargs)
    fully_shard(model, **kwargs)
    for layer in model.layers:
        fsdp2.patch_lazy_init(layer)
    fsdp2.patch_lazy_init(model)
    fully_shard.state(model)._lazy_init()  # moves the shards into the symmetric arena
    comm_ctx = fully_shard.state(model)._comm_ctx
    for s in (comm_ctx.all_gather_copy_in_stream, comm_ctx.all_gather_stream, comm_ctx.reduce_scatter_stream):
        assert s.priority == 0  # the patch keeps every stream that carries work at the default priority
    for module in [*model.layers, model]:
        fsdp2.fill_peer_shards(module, full_params)
    breakdown = fsdp2.get_symm_buffer_memory_breakdown()
    assert set(breakdown) >= {"fsdp_params", "accumulation"}
    conversions = []
    convert = fsdp2.get_gather_service().convert_symm_buffer
    fsdp2.get_gather_service().convert_symm_buffer = lambda *a, **k: (conversions.append(a), convert(*a, **k))[1]
    # rank 0's shard of every parameter is chunk 0 of the full parameter, living in the arena
    for name, p in model.named_parameters():
        local = p._local_tensor
        rows = math.ceil(full_params[name].shape[0] / W)
        assert_bit_equal(local, full_params[name][:rows], f"local shard of {name}")
        arena = __import__("odc_amd").primitives.utils.get_world().arena
        assert arena.locate(local.data_ptr())[0] == 0  # it lives in rank 0's region of the arena

    compute_dtype = torch.bfloat16 if mixed else torch.float32
    ref_compute = copy.deepcopy(reference).to(compute_dtype)
    M = 3
    g = torch.Generator().manual_seed(1)
    batches = [torch.randn(16, 32, generator=g).cuda() for _ in range(M)]

    fsdp2.pre_minibatch_start(model)
    want = {name: torch.zeros(p.numel()) for name, p in full_params.items()}
    for x in batches:
        model(x).float().pow(2).mean().backward()
        ref_compute.zero_grad(set_to_none=True)
        ref_compute(x.to(compute_dtype)).float().pow(2).mean().backward()
        for name, p in ref_compute.named_parameters():
            want[name].add_(p.grad.detach().cpu().reshape(-1))  # fp32 += compute-dtype grad, in order
    fsdp2.pre_optimizer_step(model)

    for name, p in model.named_parameters():
        rows = math.ceil(full_params[name].shape[0] / W)
        local_rows = min(rows, full_params[name].shape[0])
        rest = full_params[name][0].numel() if full_params[name].dim() > 1 else 1
        expect = oracle.fsdp2_average(want[name][: local_rows * rest].clone(), W).view(p._local_tensor.shape)
        got = p.grad._local_tensor
        assert got.dtype == torch.float32 and got.shape == expect.shape
        assert_bit_equal(got, expect, f"sharded gradient of {name}")

    # the optimizer updates rank 0's shards in place, i.e. inside the arena; the next gather sees them
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    before = {name: p._local_tensor.clone() for name, p in model.named_parameters()}
    opt.step()
    for name, p in model.named_parameters():
        assert_bit_equal(
            p._local_tensor, torch.add(before[name], p.grad._local_tensor, alpha=-0.1), f"updated shard of {name}"
        )
    updated = {name: p._local_tensor.clone() for name, p in model.named_parameters()}
    opt.zero_grad()
    fsdp2.pre_minibatch_start(model)
    out = model(batches[0])
    # reference with chunk 0 of every parameter updated and the other chunks unchanged
    with torch.no_grad():
        for name, p in reference.named_parameters():
            rows = math.ceil(p.shape[0] / W)
            p[:rows] = updated[name]
    want_out = copy.deepcopy(reference).to(compute_dtype)(batches[0].to(compute_dtype))
    assert_bit_equal(out, want_out, "forward after the optimizer step")
    # one conversion per group and minibatch, however many gathers (forward and backward, M microbatches)
    n_groups = len(model.layers) + 1
    assert len(conversions) == (2 * n_groups if mixed == "compute-dtype shards" else 0)
    if mixed == "compute-dtype shards":
        # an in-place update of the sharded parameters with no hook in between (a checkpoint
        # load, say): torch's version counters tell the copies that they are out of date
        model.reshard()
        with torch.no_grad():
            for p in model.parameters():
                p.mul_(0.5)
            for p in reference.parameters():
                p[: math.ceil(p.shape[0] / W)].mul_(0.5)
        out = model(batches[1])
        want_out = copy.deepcopy(reference).to(compute_dtype)(batches[1].to(compute_dtype))
        assert_bit_equal(out, want_out, "forward after an in-place update without a hook")
        assert len(conversions) == 3 * n_groups


@pytest.mark.parametrize("extra", [
    ["--world-size", "12", "--layers", "3", "--mixed-precision"],
    ["--world-size", "12", "--layers", "3", "--mixed-precision", "--explicit-prefetching"],
    ["--world-size", "8", "--layers", "2"],
    ["--world-size", "12", "--layers", "3", "--mixed-precision", "--no-reshard-after-forward"],
    ["--world-size", "12", "--layers", "2", "--mixed-precision", "--microbatches", "4", "--sync-every", "2"],
    ["--world-size", "12", "--layers", "2", "--mixed-precision", "--reduce-dtype", "fp16", "--microbatches", "4",
     "--sync-every", "2"],  # pre- and post-divide around fp16 accumulations
    ["--world-size", "8", "--layers", "2", "--mixed-precision", "--reduce-dtype", "bf16", "--microbatches", "3"],
    ["--world-size", "12", "--layers", "3", "--mixed-precision", "--explicit-prefetching",
     "ENV:ODC_FSDP2_COMPUTE_DTYPE_SHARDS=1"],  # gathers read a bf16 copy of the shards, renewed every step
])
def test_transformer_example_trains_bit_exactly(extra):
    """examples/fsdp2_toy.py (the counterpart of examples/FSDP2/example.py): a small transformer
    under implicit and explicit prefetching; every step's gradient shards must equal the
    unsharded model's. The first case once failed when the gathered parameters were written, from
    the prefetching stream, into storage taken from the compute stream's pool."""
    import subprocess
    import sys
    from pathlib import Path

    script = Path(__file__).resolve().parent.parent / "examples" / "fsdp2_toy.py"
    import os

    env = dict(os.environ)
    env.update(e[4:].split("=", 1) for e in extra if e.startswith("ENV:"))
    args = [e for e in extra if not e.startswith("ENV:")]
    proc = subprocess.run([sys.executable, str(script), "--steps", "4", *args],
                          capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert proc.stdout.count("match the unsharded model bit for bit") == 4


def test_frozen_and_unused_parameters_get_no_gradient(make_world, fake_process_group):
    """A group whose gradients cover only part of its accumulation (one parameter frozen, one
    module never called): the rest is reduced exactly, the two keep ``grad is None`` as under
    torch's own FSDP, and the partial cover takes the clear + accumulate route of lazy clears."""
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.fsdp import fully_shard

    from odc_amd.fsdp import fsdp2

    W = 4
    fake_process_group(W)
    mesh = init_device_mesh("cuda", (W,))
    make_world(W, 64 << 20)
    fsdp2.patch_fsdp2()
    torch.manual_seed(0)
    model = Toy().cuda()
    model.spare = nn.Linear(7, 5).cuda()  # never used in forward
    model.layers[1].up.bias.requires_grad_(False)
    reference = copy.deepcopy(model)
    full_params = {name: p.detach().clone() for name, p in reference.named_parameters()}
    for layer in model.layers:
        fully_shard(layer, mesh=mesh)
    fully_shard(model, mesh=mesh)
    for layer in model.layers:
        fsdp2.patch_lazy_init(layer)
    fsdp2.patch_lazy_init(model)
    fully_shard.state(model)._lazy_init()
    for module in [*model.layers, model]:
        fsdp2.fill_peer_shards(module, full_params)

    g = torch.Generator().manual_seed(5)
    batches = [torch.randn(16, 32, generator=g).cuda() for _ in range(2)]
    for minibatch in range(2):  # the second one starts from accumulations that hold old sums
        fsdp2.pre_minibatch_start(model)
        want = {name: torch.zeros(p.numel()) for name, p in full_params.items()}
        for x in batches:
            model(x).pow(2).mean().backward()
            reference.zero_grad(set_to_none=True)
            reference(x).pow(2).mean().backward()
            for name, p in reference.named_parameters():
                if p.grad is not None:
                    want[name].add_(p.grad.detach().cpu().reshape(-1))
        fsdp2.pre_optimizer_step(model)
        for name, p in model.named_parameters():
            if name.startswith("spare.") or name == "layers.1.up.bias":
                assert p.grad is None, name
                continue
            rows = math.ceil(full_params[name].shape[0] / W)
            rest = full_params[name][0].numel() if full_params[name].dim() > 1 else 1
            expect = oracle.fsdp2_average(want[name][: rows * rest].clone(), W).view(p._local_tensor.shape)
            assert_bit_equal(p.grad._local_tensor, expect, f"minibatch {minibatch}: sharded gradient of {name}")
        model.zero_grad(set_to_none=True)


def test_llama_architecture_example_checks_bit_exactly():
    """examples/llama_fsdp2.py --check: Hugging Face's Llama (GQA, RoPE, SwiGLU, RMSNorm; random
    weights, nothing downloaded) under fully_shard at W=12, every gradient shard against the
    unsharded model. Skipped where transformers is not installed."""
    pytest.importorskip("transformers")
    import subprocess
    import sys
    from pathlib import Path

    script = Path(__file__).resolve().parent.parent / "examples" / "llama_fsdp2.py"
    proc = subprocess.run(
        [sys.executable, str(script), "--check", "--hidden", "256", "--intermediate", "768", "--heads", "8",
         "--kv-heads", "2", "--vocab", "2000", "--layers", "2", "--seq", "64", "--world-size", "12", "--steps", "1"],
        capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "gradient shards match the unsharded model bit for bit" in proc.stdout


@pytest.mark.parametrize("mixed", [True, False])
def test_patched_equals_torch_fully_shard_at_world_size_one(make_world, mixed):
    """The reference checks its FSDP2 patches by comparing a hash of the gradients with an
    unpatched run (examples/FSDP2/utils.py:29-66, example.py). At world size 1 torch's own
    collectives move real data on one GPU (a one-rank RCCL group), so the same comparison runs
    here: two minibatches of three microbatches through torch's fully_shard as it is and through
    the patched one, equal gradient shards and equal parameters after each optimizer step."""
    import socket

    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.fsdp import MixedPrecisionPolicy, fully_shard

    from odc_amd.fsdp import fsdp2

    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    dist.init_process_group("nccl", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1,
                            device_id=torch.device("cuda", 0))
    try:
        mesh = init_device_mesh("cuda", (1,))
        torch.manual_seed(3)
        base = Toy(dim=192, hidden=300).cuda()
        kwargs = {"mesh": mesh}
        if mixed:
            kwargs["mp_policy"] = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32)
        g = torch.Generator().manual_seed(4)
        minibatches = [[torch.randn(16, 32, generator=g).cuda() for _ in range(3)] for _ in range(2)]

        def train(model, patched):
            for layer in model.layers:
                fully_shard(layer, **kwargs)
            fully_shard(model, **kwargs)
            if patched:
                for layer in model.layers:
                    fsdp2.patch_lazy_init(layer)
                fsdp2.patch_lazy_init(model)
            opt = torch.optim.SGD(model.parameters(), lr=0.05)
            seen = []
            for batches in minibatches:
                if patched:
                    fsdp2.pre_minibatch_start(model)
                for x in batches:
                    model(x).float().pow(2).mean().backward()
                if patched:
                    fsdp2.pre_optimizer_step(model)
                seen.append({n: p.grad._local_tensor.detach().clone() for n, p in model.named_parameters()})
                opt.step()
                opt.zero_grad()
                seen.append({n: p._local_tensor.detach().clone() for n, p in model.named_parameters()})
            return seen

        want = train(copy.deepcopy(base), patched=False)
        make_world(1, 64 << 20)
        fsdp2.patch_fsdp2()
        got = train(copy.deepcopy(base), patched=True)
        assert len(got) == len(want) == 4
        for step, (a, b) in enumerate(zip(got, want)):
            assert a.keys() == b.keys()
            for name in a:
                assert a[name].dtype == b[name].dtype and a[name].shape == b[name].shape
                # torch.equal: a gradient that is -0 in every microbatch stays -0 under torch's
                # `grad += new` and becomes +0 in an accumulation that starts from +0
                assert torch.equal(a[name], b[name]), f"{'gradient' if step % 2 == 0 else 'parameter'} {name}, minibatch {step // 2}"
    finally:
        fsdp2.unpatch_fsdp2()
        dist.destroy_process_group()
