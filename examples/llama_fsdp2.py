#!/usr/bin/env python3
"""A Llama-architecture model (Hugging Face ``LlamaForCausalLM``, random weights, no download)
trained with torch ``fully_shard`` through the ODC primitives on ONE GPU, as rank 0 of a W-rank
"fake" mesh: what the FSDP2 caller of the path looks like at real layer shapes.

Follows the training loop of the reference's ``examples/llm_training/torch_fsdp2.py``
(:147-187 in its FSDP2 example form: ``pre_minibatch_start`` -> microbatches ->
``pre_optimizer_step`` -> optimizer) with bf16 parameters and fp32 gradient reduction
(``MixedPrecisionPolicy`` of ``examples/FSDP2/example.py:85-88``). Dataset, packing and the
chunked LM head of that example are not reproduced: the batch is random token ids.

Prints ms per microbatch for the sharded model and for the same model run unsharded on the same
GPU; the difference is what sharding over W virtual ranks costs here (gathers, gradient
scatter-accumulates and FSDP's own bookkeeping; all compute runs on this one GPU either way).
``--check`` uses the eager attention and compares every gradient shard with the unsharded model.

    python examples/llama_fsdp2.py                       # 2 layers at Llama-3-8B width
    python examples/llama_fsdp2.py --check --hidden 512 --intermediate 1536 --layers 3 --seq 128
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

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))


def timed(fn, steps):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--intermediate", type=int, default=14336)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--kv-heads", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=2)
    ap.add_argument("--microbatches", type=int, default=4)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--check", action="store_true")
    ap.add_argument("--compute-dtype-shards", action="store_true",
                    help="gather from a bf16 copy of the fp32 shards, converted once per minibatch")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="libodc_hip launch knob, e.g. cast_resident_cap=2")
    args = ap.parse_args()

    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.fsdp import MixedPrecisionPolicy, fully_shard
    from torch.testing._internal.distributed.fake_pg import FakeStore
    from transformers import LlamaConfig, LlamaForCausalLM

    import odc_amd as odc
    from odc_amd.fsdp import fsdp2

    W = args.world_size
    torch.cuda.set_device(0)
    for opt in args.option:
        name, value = opt.split("=")
        odc._native.set_option(name, int(value))
    dist.init_process_group("fake", rank=0, world_size=W, store=FakeStore())
    mesh = init_device_mesh("cuda", (W,))
    cfg = LlamaConfig(
        hidden_size=args.hidden, intermediate_size=args.intermediate, num_hidden_layers=args.layers,
        num_attention_heads=args.heads, num_key_value_heads=args.kv_heads, vocab_size=args.vocab,
        max_position_embeddings=args.seq, tie_word_embeddings=False,
        attn_implementation="eager" if args.check else "sdpa",
    )
    torch.manual_seed(0)
    with torch.device("cuda"):
        model = LlamaForCausalLM(cfg)
    n_params = sum(p.numel() for p in model.parameters())
    # 4 B shard + 4 B accumulation (+ 2 B copy of the shard) per parameter and rank, plus room for alignment
    per_param = 10 if args.compute_dtype_shards else 8
    odc.init_nvshmem(world_size=W, symmetric_size=(n_params // W) * per_param + (64 << 20))
    fsdp2.patch_fsdp2(compute_dtype_shards=args.compute_dtype_shards)
    twin = copy.deepcopy(model).bfloat16()
    for ours, theirs in zip(twin.buffers(), model.buffers()):  # FSDP leaves buffers (rotary) in fp32
        ours.data = theirs.data.clone()
    full_params = {n: p.detach().clone() for n, p in model.named_parameters()}

    mp = MixedPrecisionPolicy(param_dtype=torch.bfloat16, reduce_dtype=torch.float32)
    for layer in model.model.layers:
        fully_shard(layer, mesh=mesh, mp_policy=mp)
    fully_shard(model, mesh=mesh, mp_policy=mp)
    for layer in model.model.layers:
        fsdp2.patch_lazy_init(layer)
    fsdp2.patch_lazy_init(model)
    fully_shard.state(model)._lazy_init()
    for module in [*model.model.layers, model]:
        fsdp2.fill_peer_shards(module, full_params)
    del full_params

    gen = torch.Generator(device="cuda").manual_seed(1)
    batches = [torch.randint(0, args.vocab, (args.batch, args.seq), device="cuda", generator=gen)
               for _ in range(args.microbatches)]

    def sharded_minibatch(_):
        fsdp2.pre_minibatch_start(model)
        for tokens in batches:
            model(input_ids=tokens, labels=tokens).loss.backward()
        fsdp2.pre_optimizer_step(model)  # the optimizer itself is left out on both sides
        model.zero_grad(set_to_none=True)

    def unsharded_minibatch(_):
        for tokens in batches:
            twin(input_ids=tokens, labels=tokens).loss.backward()
        twin.zero_grad(set_to_none=True)

    if args.check:
        fsdp2.pre_minibatch_start(model)
        want = {n: torch.zeros(p.shape, device="cuda") for n, p in twin.named_parameters()}
        for tokens in batches:
            model(input_ids=tokens, labels=tokens).loss.backward()
            twin.zero_grad(set_to_none=True)
            twin(input_ids=tokens, labels=tokens).loss.backward()
            for n, p in twin.named_parameters():
                want[n].add_(p.grad)
        fsdp2.pre_optimizer_step(model)
        for n, p in model.named_parameters():
            rows = math.ceil(want[n].shape[0] / W)
            expect = (want[n][:rows].cpu() / W).cuda()
            got = p.grad._local_tensor
            if not torch.equal(got.view(torch.int32), expect.view(torch.int32)):
                raise SystemExit(f"gradient shard of {n} differs from the unsharded model "
                                 f"(max |d| {(got - expect).abs().max().item():g})")
        print(f"{len(want)} gradient shards match the unsharded model bit for bit "
              f"({args.microbatches} microbatches, W={W})")
        model.zero_grad(set_to_none=True)
        twin.zero_grad(set_to_none=True)

    sharded_minibatch(0)  # warm-up: lazy registration, allocator, kernel selection
    unsharded_minibatch(0)
    t_sharded = timed(sharded_minibatch, args.steps) / args.microbatches
    t_plain = timed(unsharded_minibatch, args.steps) / args.microbatches
    tokens = args.batch * args.seq
    layer_params = sum(p.numel() for p in twin.model.layers[0].parameters())
    # per microbatch: every decoder layer is gathered twice (forward, backward; fp32 shards -> bf16,
    # 6 B per element) and scatter-accumulated once (10 B); the root group (embedding, final norm,
    # lm_head) stays unsharded after its forward gather, so it is gathered once
    root_params = n_params - args.layers * layer_params
    path_bytes = args.layers * layer_params * (2 * 6 + 10) + root_params * (6 + 10)
    if args.compute_dtype_shards:  # gathers move 4 B per element; the copy (6 B) is made once per minibatch
        path_bytes = (args.layers * layer_params * (2 * 4 + 10) + root_params * (4 + 10)
                      + 6 * n_params // args.microbatches)
    print(f"Llama {args.layers} x ({args.hidden}, {args.intermediate}) + vocab {args.vocab}: {n_params / 1e6:.0f} M parameters, "
          f"W={W}, {tokens} tokens per microbatch")
    print(f"sharded through ODC : {t_sharded * 1e3:8.2f} ms per microbatch  ({tokens / t_sharded:,.0f} tokens/s)")
    print(f"unsharded, same GPU : {t_plain * 1e3:8.2f} ms per microbatch  ({tokens / t_plain:,.0f} tokens/s)")
    t_path = path_bytes / 6.2e12
    print(f"difference          : {(t_sharded - t_plain) * 1e3:8.2f} ms; the gathers and "
          f"scatter-accumulates alone move {path_bytes / 1e9:.2f} GB = {t_path * 1e3:.2f} ms at 6.2 TB/s")
    from odc_amd.primitives.utils import launch_stream_policy

    print(f"hidden behind compute (ODC_COMM_STREAM={launch_stream_policy()}): "
          f"{max(0.0, 1.0 - (t_sharded - t_plain) / t_path):.0%} of that time "
          "(1 - difference / path time; FSDP's own bookkeeping counts against it)")
    fsdp2.stop()
    fsdp2.unpatch_fsdp2()
    odc.finalize_distributed()
    dist.destroy_process_group()


if __name__ == "__main__":
    main()
