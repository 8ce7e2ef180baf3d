#!/usr/bin/env python3
"""Gather micro-benchmark and self-check on one MI355X with W virtual ranks.

Same experiment as the reference's examples/all_gather.py (:49-57,80-125): `cnt` int64 tensors of
16 Mi elements, tensor i on rank r filled with i + 2r, each gathered and checked block by block
against 2r + i. The reference prints the network payload rate; with every rank in one HBM there is
no network, so this prints HBM bytes moved (read + write) per second instead.

    python examples/all_gather.py [--world-size 8] [--cnt 20] [--size 16777216]
"""

import argparse
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import torch  # noqa: E402

import odc_amd as odc  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--cnt", type=int, default=20)
    ap.add_argument("--size", type=int, default=16 * 2**20)
    args = ap.parse_args()
    W, cnt, size, dtype = args.world_size, args.cnt, args.size, torch.int64
    group = odc.init_nvshmem(world_size=W, symmetric_size=cnt * size * dtype.itemsize + (1 << 20))
    registry = odc.SymmBufferRegistry.get_instance()
    gather = odc.GatherService()
    try:
        for i in range(cnt):
            for r in range(W):
                with odc.virtual_rank(r):
                    registry.update_symm_buffer(i, torch.full((size,), i + 2 * r, dtype=dtype, device="cuda"))
        dst = torch.empty(size * W, dtype=dtype, device="cuda")
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(cnt):
            if i == 1:  # the first call warms up, as in the reference
                start.record()
            gather.gather_into_tensor(dst, registry.get_symm_buffer(i), group)
            for r in range(W):
                assert torch.eq(dst[r * size : (r + 1) * size], 2 * r + i).all(), f"tensor {i} block {r}"
        end.record()
        torch.cuda.synchronize()
        # timed again without the checks in between
        start.record()
        for i in range(cnt):
            gather.gather_into_tensor(dst, registry.get_symm_buffer(i), group)
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end)
        moved = 2 * cnt * W * size * dtype.itemsize
        print(f"gather_into_tensor: {cnt} x {W * size * dtype.itemsize / 2**20:.0f} MiB checked; "
              f"{moved / ms / 1e6:.0f} GB/s of HBM traffic ({ms / cnt * 1e3:.1f} us per gather)")
    finally:
        torch.cuda.synchronize()
        registry.finalize()
        odc.finalize_distributed()


if __name__ == "__main__":
    main()
