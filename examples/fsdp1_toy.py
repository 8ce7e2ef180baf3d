#!/usr/bin/env python3
"""The toy transformer of ``fsdp2_toy.py`` under torch's ``FullyShardedDataParallel`` (FSDP1,
flat parameters) through the ODC primitives, on ONE GPU as rank 0 of a W-rank "fake" group.

The order of calls is that of the reference's ``examples/llm_training/torch_fsdp.py``
(``patch_fsdp1(reduce_dtype=fp32)`` :59 before wrapping; per minibatch ``pre_minibatch_start``,
the microbatches, ``pre_optimizer_step`` :336-337, the optimizer). An unsharded copy of the model
runs beside it; rank 0's flat gradient shards must equal it bit for bit at every step.

    python examples/fsdp1_toy.py [--world-size 8] [--forward-prefetch] [--no-backward-prefetch]
"""

from __future__ import annotations

import argparse
import contextlib
import copy
import math
import sys
import time
from pathlib import Path

import torch
import torch.distributed as dist
import torch.nn.functional as F

sys.path.insert(0, str(Path(__file__).resolve().parent))
sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

from fsdp2_toy import Block, ToyLM  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--microbatches", type=int, default=2)
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--forward-prefetch", action="store_true")
    ap.add_argument("--no-backward-prefetch", action="store_true")
    ap.add_argument("--sync-every", type=int, default=1,
                    help="reduce gradients only every so many microbatches (no_sync() in between: the "
                         "unsharded bf16 gradients add up in place)")
    ap.add_argument("--shard-grad-op", action="store_true", help="ZeRO-2: keep parameters unsharded between forward and backward")
    args = ap.parse_args()

    from torch.distributed.fsdp import BackwardPrefetch, MixedPrecision, ShardingStrategy
    from torch.distributed.fsdp import FullyShardedDataParallel as FSDP
    from torch.distributed.fsdp._common_utils import clean_tensor_name
    from torch.distributed.fsdp.wrap import ModuleWrapPolicy
    from torch.testing._internal.distributed.fake_pg import FakeStore

    import odc_amd as odc
    from odc_amd.fsdp import fsdp1

    W = args.world_size
    torch.cuda.set_device(0)
    dist.init_process_group("fake", rank=0, world_size=W, store=FakeStore())
    odc.init_nvshmem(world_size=W, symmetric_size="1G")
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)  # bf16 gradients into fp32 accumulations

    torch.manual_seed(0)
    vocab, seq, batch = 1024, 64, 32
    model = ToyLM(vocab=vocab, seq=seq, layers=args.layers).cuda()
    unsharded = copy.deepcopy(model)
    fsdp_model = FSDP(
        model,
        auto_wrap_policy=ModuleWrapPolicy({Block}),
        mixed_precision=MixedPrecision(param_dtype=torch.bfloat16),
        device_id=torch.cuda.current_device(),
        use_orig_params=False,
        forward_prefetch=args.forward_prefetch,
        sharding_strategy=ShardingStrategy.SHARD_GRAD_OP if args.shard_grad_op else ShardingStrategy.FULL_SHARD,
        backward_prefetch=None if args.no_backward_prefetch else BackwardPrefetch.BACKWARD_PRE,
    )
    units = []  # (flat-parameter handle, names of the original parameters in flat order)
    for name, module in fsdp_model.named_modules():
        if isinstance(module, FSDP) and module._handle is not None:
            prefix = clean_tensor_name(name)
            units.append((module._handle, [f"{prefix}.{f}" if prefix else f for f in module._handle.flat_param._fqns]))
    pre, post = fsdp_model._gradient_predivide_factor, fsdp_model._gradient_postdivide_factor

    optim = torch.optim.Adam(fsdp_model.parameters(), lr=1e-3)
    data = torch.Generator(device="cuda").manual_seed(1)
    named = dict(unsharded.named_parameters())
    t0 = time.perf_counter()
    for step in range(args.steps):
        fsdp1.pre_minibatch_start(fsdp_model)
        # the unsharded twin follows rank 0's chunk of every flat parameter (what the optimizer
        # of this process updates); the other chunks stay as they were
        with torch.no_grad():
            for handle, fqns in units:
                flat = torch.cat([named[f].reshape(-1) for f in fqns])
                chunk = math.ceil(flat.numel() / W)
                flat[:chunk] = handle.flat_param.data[: min(chunk, flat.numel())]
                off = 0
                for f in fqns:
                    named[f].copy_(flat[off : off + named[f].numel()].view_as(named[f]))
                    off += named[f].numel()
        twin = copy.deepcopy(unsharded).bfloat16()
        want = [None] * len(units)
        twin.zero_grad(set_to_none=True)
        for m in range(args.microbatches):
            sync = (m + 1) % args.sync_every == 0 or m + 1 == args.microbatches
            tokens = torch.randint(0, vocab, (batch, seq), device="cuda", generator=data)
            with contextlib.nullcontext() if sync else fsdp_model.no_sync():
                loss = F.cross_entropy(fsdp_model(tokens).float().view(-1, vocab), tokens.view(-1))
                loss.backward()
            # the twin's gradients add up in bf16 between reductions, as the unsharded flat gradient does
            F.cross_entropy(twin(tokens).float().view(-1, vocab), tokens.view(-1)).backward()
            if not sync:
                continue
            grads = dict(twin.named_parameters())
            for u, (handle, fqns) in enumerate(units):
                flat_grad = torch.cat([grads[f].grad.reshape(-1) for f in fqns])
                if pre > 1:
                    flat_grad.div_(pre)  # in bf16, as torch does before the reduce-scatter
                chunk = math.ceil(flat_grad.numel() / W)
                mine = flat_grad[:chunk].float()
                want[u] = (torch.zeros_like(mine) if want[u] is None else want[u]) + mine  # first add is +0 + g
            twin.zero_grad(set_to_none=True)
        fsdp1.pre_optimizer_step(fsdp_model)
        for u, (handle, fqns) in enumerate(units):
            expect = want[u]
            if post > 1:
                expect = (expect.cpu() / post).cuda()  # the host's division is the correctly rounded one
            got = handle.flat_param.grad
            if not torch.equal(got.view(torch.int32), expect.view(torch.int32)):
                worst = (got - expect).abs().max().item()
                raise SystemExit(f"step {step}: flat gradient shard of {fqns[0]}... differs from the unsharded model (max |d| {worst:g})")
        optim.step()
        optim.zero_grad()
        print(f"step {step} loss {loss.item():.4f}  flat gradient shards match the unsharded model bit for bit")
    torch.cuda.synchronize()
    used = odc.SymmBufferRegistry.get_instance().memory_allocated()
    print(f"{args.steps} steps in {time.perf_counter() - t0:.2f} s; symmetric memory per rank: {used / 2**20:.1f} MiB")
    fsdp1.stop()
    fsdp1.unpatch_fsdp1()
    odc.finalize_distributed()
    dist.destroy_process_group()


if __name__ == "__main__":
    main()
