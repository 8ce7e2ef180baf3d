#!/usr/bin/env python3
"""Scatter-accumulate micro-benchmark and self-check on one MI355X with W virtual ranks.

Same experiment as the reference's examples/reduce_scatter.py (:49-56,96-105,163-172): every rank
contributes `times` random fp32 gradients of 128 Mi + 1024 elements; the accumulations are compared
with reduce-scatter(sum) + add_ within rtol = atol = 5e-3. Here the W ranks are virtual (one after
the other on one GPU), the reduce-scatter reference is computed with torch on the same device, and
the rate printed is HBM bytes moved (gradient read + accumulation read and write) per second.

    python examples/reduce_scatter.py [--world-size 8] [--times 4] [--size 134218752] [--grad-dtype fp32|bf16]
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
    ap.add_argument("--times", type=int, default=4)
    ap.add_argument("--size", type=int, default=128 * 1024**2 + 1024)
    ap.add_argument("--grad-dtype", choices=["fp32", "bf16"], default="fp32")
    args = ap.parse_args()
    W, times, size = args.world_size, args.times, args.size
    assert size % W == 0, "the gradient must split evenly over the ranks (scatter_accumulate.py:589-592)"
    grad_dtype = torch.float32 if args.grad_dtype == "fp32" else torch.bfloat16
    group = odc.init_nvshmem(world_size=W, symmetric_size=size // W * 4 + (1 << 20))
    registry = odc.SymmBufferRegistry.get_instance()
    service = odc.ReductionService(accumulation_dtype=torch.float32)
    try:
        expected = torch.zeros(size, dtype=torch.float32, device="cuda")
        gen = torch.Generator(device="cuda").manual_seed(0)
        service.scatter_accumulate(0, torch.zeros(size, dtype=grad_dtype, device="cuda"), group)  # registers
        service.clear_accumulations()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        elapsed_ms = 0.0
        for _ in range(times):
            grads = [torch.rand(size, generator=gen, device="cuda").to(grad_dtype) for _ in range(W)]
            start.record()
            for q in range(W):  # every virtual rank is a client, in rank order
                with odc.virtual_rank(q):
                    service.scatter_accumulate(0, grads[q], group)
            end.record()
            torch.cuda.synchronize()
            elapsed_ms += start.elapsed_time(end)
            expected.add_(torch.stack([g.float() for g in grads]).sum(0))  # reduce_scatter(sum) + add_
        service.sync(group)
        for r, acc in enumerate(service.get_peer_accumulations(0)):
            torch.testing.assert_close(acc, expected.view(W, -1)[r], rtol=5e-3, atol=5e-3)
        moved = times * W * size * (grad_dtype.itemsize + 8)
        print(f"scatter_accumulate: {times} rounds x {W} clients of {size} {args.grad_dtype} elements match "
              f"reduce-scatter + add; {moved / elapsed_ms / 1e6:.0f} GB/s of HBM traffic "
              f"({elapsed_ms / (times * W) * 1e3:.1f} us per call)")
    finally:
        torch.cuda.synchronize()
        registry.finalize()
        odc.finalize_distributed()


if __name__ == "__main__":
    main()
