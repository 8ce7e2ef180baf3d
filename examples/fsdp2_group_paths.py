#!/usr/bin/env python3
"""What folding FSDP2's copy-in / copy-out, the dtype conversion and the end-of-minibatch divide
into the kernels saves, measured on one FSDP2 parameter group = one Llama-3-8B decoder layer
(9 parameters, fp32 master shards, bf16 compute, fp32 gradient reduction), W virtual ranks.

Per operation the reference's data flow (``fused=False``) is timed against the fused one:

    unshard   gather fp32 [W, sum n_p] + split_with_sizes_copy + cast to bf16
              (odc/fsdp/fsdp2.py:254-313, 378-401, 341-343)          vs  one converting gather
    reduce    chunk_cat of bf16 gradients into fp32 [W, sum n_p] + scatter-accumulate
              (odc/fsdp/fsdp2.py:671-682, 708-710)                   vs  one scatter-accumulate
    publish   acc /= W, then acc.to(bf16) (odc/fsdp/fsdp2.py:846-847, 897-899) vs  one pass
    clear     acc.fill_(0) per rank (odc/primitives/scatter_accumulate.py:585-587) vs  one launch

Both flows are bit-identical (tests/test_gpu_fsdp.py); this script only times them.

    python examples/fsdp2_group_paths.py [--world-size 8]
"""

from __future__ import annotations

import argparse
import statistics
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one torch copy of 1 GiB (counter calibration under rocprofv3)")
    ap.add_argument("--publish-groups", type=int, default=0, metavar="K",
                    help="also time the publish of K layer-sized accumulations in ONE launch "
                         "(what pre_optimizer_step does for a model's parameter groups)")
    ap.add_argument("--compute-dtype-shards", action="store_true",
                    help="also time the unshard from a bf16 copy of the shards (converted once per "
                         "minibatch) and that conversion")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="a launch knob of the library, e.g. cast_resident_cap=4")
    args = ap.parse_args()

    import odc_amd as odc
    from odc_amd import _native

    for opt in args.option:
        name, _, value = opt.partition("=")
        _native.set_option(name, int(value))
    from odc_amd.fsdp import fsdp2
    from odc_amd.workloads import llama3_8b_layer_shapes, numel

    W = args.world_size
    torch.cuda.set_device(0)
    shapes = [s for _, s in llama3_8b_layer_shapes()]
    N = sum(numel(s) for s in shapes)
    group = odc.init_nvshmem(world_size=W, symmetric_size=(N // W) * (16 + 4 * args.publish_groups + 8 * args.compute_dtype_shards) + (64 << 20))
    fsdp2.patch_fsdp2()  # creates the two services the group uses (nothing of torch is touched here)
    layer = fsdp2.ParamGroup(shapes, torch.float32, group, param_dtype=torch.bfloat16,
                             reduce_dtype=torch.float32, name="layer")
    gen = torch.Generator(device="cuda").manual_seed(0)
    layer.load_full_params([torch.randn(s, generator=gen, device="cuda") * 0.02 for s in shapes])
    grads = [(torch.randn(s, generator=gen, device="cuda") * 1e-3).bfloat16() for s in shapes]
    side = torch.cuda.Stream()

    def timed(fn):
        with torch.cuda.stream(side):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            samples = []
            for _ in range(5):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(side)
                for _ in range(args.iters):
                    fn()
                e1.record(side)
                e1.synchronize()
                samples.append(e0.elapsed_time(e1) / args.iters)
        return statistics.median(samples)

    def unshard(fused):
        layer.unshard(fused=fused)
        layer.reshard()

    scatter = fsdp2.get_reduction_service()
    scatter.lazy_clear = False  # every timed reduce is the read-modify-write
    layer.reduce(grads)  # registers the accumulation

    def publish_reference():
        acc = scatter.get_accumulation(id(layer))
        acc /= W
        return acc.to(torch.bfloat16)

    def publish_fused():
        return scatter.publish([id(layer)], out_dtype=torch.bfloat16, divisor=float(W))

    unshard_row = ("unshard (fp32 shards -> bf16 parameters)", timed(lambda: unshard(False)), timed(lambda: unshard(True)), 6 * N)
    fused_reduce = timed(lambda: layer.reduce(grads, fused=True))
    publish_row = ("publish (acc /= W, bf16 copy; one rank)", timed(publish_reference), timed(publish_fused), 10 * N // W)
    clear_row = ("clear (zero the fp32 accumulations of all ranks)",
                 timed(lambda: [a.zero_() for a in scatter.get_peer_accumulations(id(layer))]),
                 timed(scatter.clear_accumulations), 4 * N)
    # The two-step flow lays its accumulation out like the reduce-scatter output (packed); the
    # fused one starts every slice on a tile. A group does one or the other, so the reference flow
    # gets a group of its own (created last: the clear above covers one accumulation only).
    reference_layer = fsdp2.ParamGroup(shapes, torch.float32, group, param_dtype=torch.bfloat16,
                                       reduce_dtype=torch.float32, name="layer, two-step reduce")
    rows = [
        unshard_row,
        ("reduce (bf16 gradients -> fp32 accumulations)", timed(lambda: reference_layer.reduce(grads, fused=False)),
         fused_reduce, 10 * N),
        publish_row,
        clear_row,
    ]
    if args.calibrate:
        a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()
    print(f"Llama-3-8B layer as one FSDP2 group: {N} parameters, W={W}")
    print(f"{'':48s} {'reference flow':>15s} {'fused':>10s} {'fused GB/s':>11s}")
    for name, ref_ms, fused_ms, fused_bytes in rows:
        print(f"{name:48s} {ref_ms * 1e3:12.1f} us {fused_ms * 1e3:7.1f} us {fused_bytes / fused_ms / 1e6:11.0f}")
    if args.publish_groups:
        keys = [("extra group", k) for k in range(args.publish_groups)]
        for key in keys:
            scatter.register(key, (N // W,), torch.bfloat16, torch.float32, group)
        ms = timed(lambda: scatter.publish(keys, out_dtype=torch.bfloat16, divisor=float(W)))
        moved = 10 * (N // W) * len(keys)
        print(f"publish of {len(keys)} such groups in one launch: {ms * 1e3:.1f} us, {moved / ms / 1e6:.0f} GB/s")
    if args.compute_dtype_shards:
        kept = fsdp2.ParamGroup(shapes, torch.float32, group, param_dtype=torch.bfloat16,
                                name="layer, bf16 copy of the shards", compute_dtype_shards=True)
        kept.load_full_params([torch.randn(s, generator=gen, device="cuda") * 0.02 for s in shapes])

        def unshard_kept():
            kept.unshard()
            kept.reshard()

        unshard_kept()  # makes the copy
        gather_ms = timed(unshard_kept)
        convert_ms = timed(lambda: fsdp2.get_gather_service().convert_symm_buffer(kept.key + "_as_bfloat16", kept.key))
        print(f"unshard from a bf16 copy of the shards: {gather_ms * 1e3:.1f} us ({4 * N / gather_ms / 1e6:.0f} GB/s); "
              f"making the copy, once per minibatch, all {W} ranks' shards: {convert_ms * 1e3:.1f} us "
              f"({6 * N / convert_ms / 1e6:.0f} GB/s)")
    torch.cuda.synchronize()
    fsdp2.stop()
    odc.finalize_distributed()


if __name__ == "__main__":
    main()
