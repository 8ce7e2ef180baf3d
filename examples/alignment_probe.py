#!/usr/bin/env python3
"""What a misaligned buffer costs the streaming kernels on this GPU.

One scatter-accumulate (bf16 gradient into an fp32 accumulation, read-modify-write) and one gather
of a buffer too large for the last-level cache, with the accumulation slice, the gradient, the
shard slice and the output each shifted by 0 ... 16 KiB. On MI355X the read-modify-write loses up
to 5.5 % when its 16 KiB tiles start 8 KiB past a 16 KiB boundary of the ACCUMULATION and nothing
when the gradient is shifted; the gather loses about 1 % per shifted side. This is why the arena
and the FSDP2 group layout start buffers and slices on tile boundaries.

    python examples/alignment_probe.py [--world-size 8] [--repeats 9]
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
    ap.add_argument("--repeats", type=int, default=9)
    ap.add_argument("--launches", type=int, default=20, help="launches per timed interval")
    args = ap.parse_args()

    import odc_amd as odc

    W = args.world_size
    torch.cuda.set_device(0)
    n_acc = 6656 * 4096  # elements per rank of the accumulate: 109 MB of fp32 per rank
    n_gat = 2 * n_acc    # bf16 elements per rank of the gather: 109 MB per rank
    slack = 16384
    group = odc.init_nvshmem(world_size=W, symmetric_size=(n_acc + slack) * 4 + (n_gat + slack) * 2 + (8 << 20))
    registry = odc.SymmBufferRegistry.get_instance()
    gather, reduction = odc.GatherService(), odc.ReductionService(accumulation_dtype=torch.float32)

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        samples = []
        for _ in range(args.repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.launches):
                fn()
            e1.record()
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) / args.launches)
        return statistics.median(samples)

    shifts = (0, 2048, 4096, 8192, 12288, 16384)
    host_side = torch.empty(W * n_gat * 2 + (1 << 20), dtype=torch.uint8, device="cuda")  # gradient, then output
    host_side.view(torch.bfloat16).normal_(0, 1e-3)

    reduction.register("acc", (n_acc + slack,), torch.bfloat16, torch.float32, group)
    print(f"scatter-accumulate, {W} x {n_acc} elements, GB/s by byte shift of the slice in the accumulation (rows) "
          f"and of the gradient (columns)")
    print(f"{'':>8s}" + "".join(f"{g:>8d}" for g in shifts))
    for a in shifts:
        row = []
        for g in shifts:
            grad = host_side[g:g + W * n_acc * 2].view(torch.bfloat16)
            ms = timed(lambda: reduction.scatter_accumulate_slices("acc", [grad], [a // 4], [n_acc], group))
            row.append(10 * W * n_acc / ms / 1e6)
        print(f"{a:>8d}" + "".join(f"{x:8.0f}" for x in row), flush=True)

    shards = registry.allocate_symm_buffer("shards", (n_gat + slack,), torch.bfloat16)
    print(f"gather, {W} x {n_gat} bf16 elements, GB/s by byte shift of the shard slice (rows) and of the output (columns)")
    print(f"{'':>8s}" + "".join(f"{d:>8d}" for d in shifts))
    for s in shifts:
        row = []
        for d in shifts:
            out = host_side[d:d + W * n_gat * 2].view(torch.bfloat16)
            ms = timed(lambda: gather.gather_slices([out], shards, [s // 2], [n_gat], group))
            row.append(4 * W * n_gat / ms / 1e6)
        print(f"{s:>8d}" + "".join(f"{x:8.0f}" for x in row), flush=True)
    torch.cuda.synchronize()
    registry.finalize()
    odc.finalize_distributed()


if __name__ == "__main__":
    main()
