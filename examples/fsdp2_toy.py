#!/usr/bin/env python3
"""A toy decoder-only transformer trained with torch's ``fully_shard`` (FSDP2) through the ODC
primitives, on ONE GPU: the process is rank 0 of a W-rank mesh over torch's "fake" process
group, and the other ranks' parameter shards are passive memory in the symmetric arena.

Counterpart of the reference's ``examples/FSDP2/example.py`` (same order of calls: init, patch,
``fully_shard`` layer by layer, ``patch_lazy_init``, then per minibatch ``pre_minibatch_start`` ->
microbatches -> ``pre_optimizer_step`` -> optimizer). Where that script compares gradient hashes
between runs (``examples/FSDP2/utils.py:29-66``), this one keeps an unsharded copy of the model
in the same process and checks rank 0's gradient shards against it bit for bit at every step.

    python examples/fsdp2_toy.py [--world-size 8] [--mixed-precision] [--explicit-prefetching]
"""

from __future__ import annotations

import argparse
import copy
import math
import sys
import time
from pathlib import Path

import torch
import torch.distributed as dist
import torch.nn as nn
import torch.nn.functional as F

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))


class Block(nn.Module):
    def __init__(self, dim, heads):
        super().__init__()
        self.heads = heads
        self.norm1 = nn.LayerNorm(dim)
        self.qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.proj = nn.Linear(dim, dim, bias=False)
        self.norm2 = nn.LayerNorm(dim)
        self.up = nn.Linear(dim, 4 * dim)
        self.down = nn.Linear(4 * dim, dim)

    def forward(self, x):
        b, t, d = x.shape
        q, k, v = self.qkv(self.norm1(x)).view(b, t, 3, self.heads, d // self.heads).permute(2, 0, 3, 1, 4)
        # the explicit-math attention: the same kernels whatever the dtype, so the sharded and
        # the unsharded model run identical arithmetic
        scores = (q @ k.transpose(-1, -2)) / math.sqrt(d // self.heads)
        causal = torch.ones(t, t, dtype=torch.bool, device=x.device).tril()
        attn = scores.masked_fill(~causal, float("-inf")).softmax(-1) @ v
        x = x + self.proj(attn.transpose(1, 2).reshape(b, t, d))
        return x + self.down(F.gelu(self.up(self.norm2(x))))


class ToyLM(nn.Module):
    def __init__(self, vocab=1024, seq=64, dim=256, heads=4, layers=2):
        super().__init__()
        self.tok = nn.Embedding(vocab, dim)
        self.pos = nn.Embedding(seq, dim)
        self.layers = nn.ModuleList([Block(dim, heads) for _ in range(layers)])
        self.norm = nn.LayerNorm(dim)
        self.out = nn.Linear(dim, vocab, bias=False)

    def forward(self, tokens):
        x = self.tok(tokens) + self.pos(torch.arange(tokens.shape[1], device=tokens.device))
        for layer in self.layers:
            x = layer(x)
        return self.out(self.norm(x))


def local_rows(full: torch.Tensor, world: int) -> torch.Tensor:
    """Rank 0's shard of ``full`` under FSDP2's dim-0 sharding."""
    return full[: math.ceil(full.shape[0] / world)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--mixed-precision", action="store_true")
    ap.add_argument("--reduce-dtype", choices=["fp32", "bf16", "fp16"], default="fp32",
                    help="with --mixed-precision: the dtype gradients are reduced and accumulated in "
                         "(fp16 splits the division by W into a pre- and a post-divide)")
    ap.add_argument("--explicit-prefetching", action="store_true")
    ap.add_argument("--no-reshard-after-forward", action="store_true",
                    help="ZeRO-2: keep parameters unsharded between forward and backward")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--microbatches", type=int, default=2)
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--sync-every", type=int, default=1,
                    help="reduce gradients only every so many microbatches (set_requires_gradient_sync); in "
                         "between they add up unsharded, in the compute dtype")
    args = ap.parse_args()

    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.fsdp import MixedPrecisionPolicy, fully_shard
    from torch.testing._internal.distributed.fake_pg import FakeStore

    import odc_amd as odc
    from odc_amd.fsdp import fsdp2

    W = args.world_size
    torch.cuda.set_device(0)
    dist.init_process_group("fake", rank=0, world_size=W, store=FakeStore())
    mesh = init_device_mesh("cuda", (W,))
    odc.init_nvshmem(world_size=W, symmetric_size="1G")
    fsdp2.patch_fsdp2()

    torch.manual_seed(0)
    vocab, seq, batch = 1024, 64, 32
    model = ToyLM(vocab=vocab, seq=seq, layers=args.layers).cuda()
    unsharded = copy.deepcopy(model)
    full_params = {n: p.detach().clone() for n, p in unsharded.named_parameters()}

    kwargs = {"mesh": mesh, "reshard_after_forward": not args.no_reshard_after_forward}
    compute_dtype = reduce_dtype = torch.float32
    if args.mixed_precision:
        reduce_dtype = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[args.reduce_dtype]
        kwargs["mp_policy"] = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=reduce_dtype)
        compute_dtype = torch.bfloat16
    # torch's rule (_fsdp_collectives._get_gradient_divide_factors): fp32 / bf16 reduce with AVG, i.e.
    # one division by W at the end; fp16 divides by ~sqrt(W) before and by the rest after
    pre_divide, post_divide = None, float(W)
    if reduce_dtype == torch.float16:
        pre_divide = 1
        while W % pre_divide == 0 and W / pre_divide > pre_divide:
            pre_divide *= 2
        post_divide = W / pre_divide

    def add_in(acc, x):
        """acc (reduce dtype) += x: computed in fp32, rounded to acc's dtype, as torch's add_ does."""
        return (acc.float() + x.float()).to(acc.dtype)
    for layer in model.layers:
        fully_shard(layer, **kwargs)
    fully_shard(model, **kwargs)
    for layer in model.layers:
        fsdp2.patch_lazy_init(layer)
    fsdp2.patch_lazy_init(model)
    fully_shard.state(model)._lazy_init()  # moves rank 0's shards into the symmetric arena
    for module in [*model.layers, model]:
        fsdp2.fill_peer_shards(module, full_params)  # what the other W-1 processes would hold
    if args.explicit_prefetching:
        for i, layer in enumerate(model.layers[:-1]):
            layer.set_modules_to_forward_prefetch([model.layers[i + 1]])
        for i, layer in enumerate(model.layers[1:], start=1):
            layer.set_modules_to_backward_prefetch([model.layers[i - 1]])

    optim = torch.optim.Adam(model.parameters(), lr=1e-3)
    names = [n for n, _ in model.named_parameters()]
    data = torch.Generator(device="cuda").manual_seed(1)
    t0 = time.perf_counter()
    for step in range(args.steps):
        fsdp2.pre_minibatch_start(model)
        # the unsharded twin sees the same parameters as the mesh does: rank 0's rows follow the
        # optimizer, the other ranks' rows stay as they were (nobody steps them in this process)
        with torch.no_grad():
            for (n, p), q in zip(model.named_parameters(), unsharded.parameters()):
                local_rows(q, W).copy_(p._local_tensor)
        twin = copy.deepcopy(unsharded).to(compute_dtype)
        if args.explicit_prefetching:
            model.unshard()
        want = {n: torch.zeros_like(full_params[n], dtype=reduce_dtype) for n in names}
        pending = {}  # gradients not reduced yet: FSDP keeps their sum unsharded, in the reduce dtype
        for m in range(args.microbatches):
            sync = (m + 1) % args.sync_every == 0 or m + 1 == args.microbatches
            model.set_requires_gradient_sync(sync)
            tokens = torch.randint(0, vocab, (batch, seq), device="cuda", generator=data)
            loss = F.cross_entropy(model(tokens).float().view(-1, vocab), tokens.view(-1))
            loss.backward()
            twin.zero_grad(set_to_none=True)
            F.cross_entropy(twin(tokens).float().view(-1, vocab), tokens.view(-1)).backward()
            for n, p in twin.named_parameters():
                pending[n] = p.grad.to(reduce_dtype) if n not in pending else add_in(pending[n], p.grad)
            if sync:
                for n in names:
                    g = pending.pop(n)
                    if pre_divide is not None and pre_divide > 1:
                        g = g / pre_divide  # a power of two: exact but for fp16 underflow
                    want[n] = add_in(want[n], g)  # what reaches the reduction, in order
        fsdp2.pre_optimizer_step(model)
        for n, p in model.named_parameters():
            got = p.grad._local_tensor
            # the last division on the host, where torch's is the correctly rounded one for every W;
            # the gradient is handed over in the parameters' own dtype (fp32)
            expect = (local_rows(want[n], W).cpu() / post_divide).float().cuda()
            if not torch.equal(got.view(torch.int32), expect.view(torch.int32)):
                worst = (got - expect).abs().max().item()
                raise SystemExit(f"step {step}: gradient shard of {n} differs from the unsharded model (max |d| {worst:g})")
        optim.step()
        optim.zero_grad()
        print(f"step {step} loss {loss.item():.4f}  gradient shards match the unsharded model bit for bit")
    torch.cuda.synchronize()
    used = odc.SymmBufferRegistry.get_instance().memory_allocated()
    print(f"{args.steps} steps in {time.perf_counter() - t0:.2f} s; symmetric memory per rank: {used / 2**20:.1f} MiB "
          f"(GB by kind: {fsdp2.get_symm_buffer_memory_breakdown()})")
    fsdp2.stop()
    fsdp2.unpatch_fsdp2()
    odc.finalize_distributed()
    dist.destroy_process_group()


if __name__ == "__main__":
    main()
