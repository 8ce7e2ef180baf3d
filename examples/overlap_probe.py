#!/usr/bin/env python3
"""How much of a gather / scatter-accumulate hides behind compute on ONE GPU.

ODC hops to a side stream so that its data movement overlaps the model's compute
(odc/primitives/gather.py:114-176, utils.py:205-209). In the reference the movement crosses
NVLink; here all W ranks live in one HBM, so the "movement" is a streaming kernel that competes
with the compute kernels for the same CUs and the same memory. This probe measures what is left
of the overlap: a chain of bf16 GEMMs (compute bound) on one stream, the layer's gather or
scatter-accumulate launches on another, alone and together.

    hidden = (t_gemm + t_path - t_both) / t_path      1 = free, 0 = fully serialised

It also compares launch shapes that matter once kernels co-reside: a residency cap on the gather
(which works by claiming LDS it never touches, so a capped gather cannot share a CU with a GEMM
that needs its LDS) and the one-workgroup-per-tile launches against persistent ones.

    python examples/overlap_probe.py [--gemm 8192] [--launches 8]
"""

from __future__ import annotations

import argparse
import sys
import time
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--world-size", type=int, default=8)
    ap.add_argument("--gemm", type=int, default=8192, help="square bf16 GEMM size of the compute chain")
    ap.add_argument("--launches", type=int, default=8, help="gather / scatter-accumulate launches per measurement")
    ap.add_argument("--repeats", type=int, default=5)
    args = ap.parse_args()

    import odc_amd as odc
    from odc_amd import _native
    from odc_amd.workloads import llama3_8b_layer_shapes, numel

    W = args.world_size
    torch.cuda.set_device(0)
    numels = [numel(s) for _, s in llama3_8b_layer_shapes()]
    N = sum(numels)
    group = odc.init_nvshmem(world_size=W, symmetric_size=sum((n // W) * 6 + 512 for n in numels) + (1 << 20))
    registry = odc.SymmBufferRegistry.get_instance()
    gather, reduction = odc.GatherService(), odc.ReductionService(accumulation_dtype=torch.float32)
    keys = list(range(len(numels)))
    shards = [registry.allocate_symm_buffer(k, (n // W,), torch.bfloat16) for k, n in zip(keys, numels)]
    for k in keys:
        for peer in registry.peer_tensors[k]:
            peer.normal_(0, 0.02)
    outs = [torch.empty(n, dtype=torch.bfloat16, device="cuda") for n in numels]
    grads = [torch.empty(n, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3) for n in numels]
    for k, n in zip(keys, numels):
        reduction.register(k, (n // W,), torch.bfloat16, torch.float32, group)

    a = torch.randn(args.gemm, args.gemm, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(args.gemm, args.gemm, device="cuda", dtype=torch.bfloat16)
    c = torch.empty_like(a)
    compute, side = torch.cuda.Stream(), torch.cuda.Stream()

    def run_gather():
        for _ in range(args.launches):
            gather.gather_into_tensors(outs, shards, group)

    def run_accum():
        for _ in range(args.launches):
            reduction.scatter_accumulate_multi(keys, grads, group)

    def one(fn_side, n_gemm):
        """Wall time of n_gemm GEMMs on `compute` and fn_side on `side`, started together."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if n_gemm:
            with torch.cuda.stream(compute):
                for _ in range(n_gemm):
                    torch.matmul(a, b, out=c)
        if fn_side is not None:
            with torch.cuda.stream(side):
                fn_side()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    def best(fn_side, n_gemm):
        one(fn_side, n_gemm)
        return min(one(fn_side, n_gemm) for _ in range(args.repeats))

    t_gemm1 = best(None, 4) / 4
    print(f"bf16 GEMM {args.gemm}^3: {t_gemm1 * 1e3:.3f} ms = {2 * args.gemm ** 3 / t_gemm1 / 1e12:.0f} TFLOP/s; "
          f"layer of {N} elements, W={W}, {args.launches} launches per measurement")
    print(f"{'path kernel, launch shape':62s} {'alone ms':>9s} {'gemm ms':>8s} {'both ms':>8s} {'hidden':>7s}")

    def report(label, fn_side, options):
        for name, value in options.items():
            _native.set_option(name, value)
        t_path = best(fn_side, 0)
        n_gemm = max(1, round(t_path / t_gemm1))  # compute of about the same length
        t_gemm = best(None, n_gemm)
        t_both = best(fn_side, n_gemm)
        hidden = (t_gemm + t_path - t_both) / t_path
        print(f"{label:62s} {t_path * 1e3:9.3f} {t_gemm * 1e3:8.3f} {t_both * 1e3:8.3f} {hidden:7.2f}")

    report("gather, one 512-thread workgroup per tile (default: 4 fit a CU)", run_gather, {"gather_resident_cap": 0})
    report("gather, one workgroup per tile, <= 2 resident per CU (LDS claim)", run_gather, {"gather_resident_cap": 2})
    report("gather, 1 persistent workgroup per CU", run_gather, {"gather_blocks_per_cu": 1})
    _native.set_option("gather_blocks_per_cu", 0)
    _native.set_option("gather_resident_cap", 0)
    report("scatter-accumulate, one workgroup per tile, no cap (default)", run_accum,
           {"accum_blocks_per_cu": 0, "accum_resident_cap": 0})
    report("scatter-accumulate, one workgroup per tile, <= 4 resident per CU", run_accum,
           {"accum_blocks_per_cu": 0, "accum_resident_cap": 4})
    report("scatter-accumulate, 1 persistent workgroup per CU", run_accum, {"accum_blocks_per_cu": 1})
    _native.set_option("accum_blocks_per_cu", -1)
    _native.set_option("accum_resident_cap", 0)
    torch.cuda.synchronize()
    registry.finalize()
    odc.finalize_distributed()


if __name__ == "__main__":
    main()
