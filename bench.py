#!/usr/bin/env python3
"""Benchmark of the ODC hot path on one MI355X: gather + scatter-accumulate over a Llama-3-8B
decoder layer sharded over W=8 virtual ranks.

One step = one microbatch of the path over the whole layer:
    gather            all 9 parameters, bf16, W shards -> full tensors      (one launch, 4N bytes)
    scatter-accumulate all 9 bf16 gradients into the W fp32 accumulations   (one launch, 10N bytes)
Every 8th step starts a new minibatch and first clears the accumulations (inside the timed
region; its 4N written bytes are NOT counted in the numerator).

Prints ONE JSON line: whole-step throughput (`value`), per-kernel roofline figures from HIP events
on the launch stream (`roofline` for the scatter-accumulate, `roofline_gather`), the clear, the
CPU oracle timed on the host cores (`cpu_baseline`), the parity verdict against that oracle, and
`other_clear_mode`: the same steps with the services' default lazy clears, where no clear kernel
runs and the first scatter-accumulate of a minibatch stores instead (6N bytes, counted as such).

Other workloads (not the headline): `--workload uneven --world-size 12` (40 uneven, zero-padded
flat parameters), `--workload model` (the whole 8.03 G-parameter model), `--layout flat`,
`--world-size 64`.
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
MICROBATCHES = 8

# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc (FETCH_SIZE and
# WRITE_SIZE runs, scaled by a torch copy kernel of known size); None until measured.
MEASURED_TRAFFIC_BYTES = {
    ("accum", "per-param", 8): 2_181_147_887,
    ("gather", "per-param", 8): 872_565_155,
    ("store", "per-param", 8): 1_308_913_261,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--world-size", type=int, default=8, help="virtual ranks W")
    ap.add_argument("--workload", choices=["layer", "uneven", "model"], default="layer",
                    help="layer: one Llama-3-8B decoder layer (the headline); uneven: 40 flat parameters of "
                         "log-uniform size, none divisible by W (run it with --world-size 12): shards are "
                         "zero padded and the gradients end before the padding; model: the full 8.03 G "
                         "parameter model swept unit by unit (needs ~85 GB of HBM; no oracle pass)")
    ap.add_argument("--layout", choices=["per-param", "flat"], default="per-param",
                    help="9 per-parameter shards in one multi-tensor launch, or one flat shard")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline sample length")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--lazy-clear", action="store_true",
                    help="the services' default mode: no clear kernel, the first scatter-accumulate of a "
                         "minibatch stores instead (6N bytes); the headline keeps eager clears so that "
                         "every timed scatter-accumulate is the 10N read-modify-write")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one torch copy of 1 GiB (counter calibration under rocprofv3)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="libodc_hip launch knob, e.g. accum_blocks_per_cu=4")
    return ap.parse_args()


def model_sweep(args):
    """Full Llama-3-8B: per step (= microbatch), gather the 34 FSDP units in forward order, then
    scatter-accumulate them in reverse order; every 8th step first clears all accumulations."""
    import torch

    import odc_amd
    from odc_amd import _native
    from odc_amd.primitives.utils import get_comm_stream
    from odc_amd.workloads import llama3_8b_units, numel

    torch.cuda.set_device(0)
    for opt in args.option:
        name, value = opt.split("=")
        _native.set_option(name, int(value))
    W = args.world_size
    units = llama3_8b_units()
    N = sum(numel(s) for _, unit in units for _, s in unit)
    per_rank = sum((numel(s) // W) * 6 + 512 for _, unit in units for _, s in unit) + (1 << 20)
    group = odc_amd.init_nvshmem(world_size=W, symmetric_size=per_rank)
    registry = odc_amd.SymmBufferRegistry.get_instance()
    gather = odc_amd.GatherService()
    reduction = odc_amd.ReductionService(accumulation_dtype=torch.float32, lazy_clear=args.lazy_clear)
    gen = torch.Generator(device="cuda").manual_seed(0)
    by_shape = {}  # unit signature -> (output buffers, two sets of gradients): reused across layers
    plan = []
    for u, (_, unit) in enumerate(units):
        sig = tuple(numel(s) for _, s in unit)
        if sig not in by_shape:
            outs = [torch.empty(n, dtype=torch.bfloat16, device="cuda") for n in sig]
            grads = [[(torch.randn(n, generator=gen, device="cuda") * 1e-3).bfloat16() for n in sig] for _ in range(2)]
            by_shape[sig] = (outs, grads)
        keys = [(u, p) for p in range(len(unit))]
        for key, n in zip(keys, sig):
            registry.allocate_symm_buffer(key, (n // W,), torch.bfloat16)
            for peer in registry.peer_tensors[key]:
                peer.normal_(0.0, 0.02, generator=gen)
            reduction.register(key, (n // W,), torch.bfloat16, torch.float32, group)
        plan.append((keys, [registry.get_symm_buffer(k) for k in keys], *by_shape[sig]))
    torch.cuda.synchronize()
    comm = get_comm_stream()

    def step(i):
        if i % MICROBATCHES == 0:
            reduction.clear_accumulations()
        for keys, locals_, outs, grads in plan:
            gather.gather_into_tensors(outs, locals_, group)
        for keys, locals_, outs, grads in reversed(plan):
            reduction.scatter_accumulate_multi(keys, grads[i % 2], group)

    gc.collect()
    gc.disable()
    with torch.cuda.stream(comm):
        for i in range(args.warmup):
            step(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(comm)
        for i in range(args.steps):
            step(i)
        e1.record(comm)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    gc.enable()
    stores = len(range(0, args.steps, MICROBATCHES)) if args.lazy_clear else 0  # 6N instead of 10N
    step_bytes = (args.steps * 14 * N - stores * 4 * N) / args.steps
    value = args.steps * step_bytes / elapsed / 1e9
    print(json.dumps({
        "metric": "achieved HBM GB/s (% of ~8 TB/s peak) for gather + scatter-accum, full 8B model sweep, W=8",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"cfg5: full Llama-3-8B ({N} bf16 params, {len(units)} units, {2 * len(units)} "
                               f"launches per step), W={W} virtual shards", "world_size": W, "elements": N,
                   "bytes_per_step": round(step_bytes),
                   "clear": "lazy (store on the first microbatch)" if args.lazy_clear else "eager"},
        "minibatch_ms": round(elapsed / args.steps * MICROBATCHES * 1e3, 3),
        "frac_of_peak": round(value / HBM_PEAK_GBPS, 4),
        "gpu_ms_per_step": round(e0.elapsed_time(e1) / args.steps, 3),
        "roofline": None, "cpu_baseline": None, "parity_vs_oracle": None,
    }))
    torch.cuda.synchronize()
    registry.finalize()
    odc_amd.finalize_distributed()


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: W virtual ranks share one MI355X and nothing here uses a "
              "second GPU. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.workload == "model":
        return model_sweep(args)

    import torch

    import odc_amd
    from odc_amd import _native
    from odc_amd.primitives.utils import get_comm_stream
    from odc_amd.workloads import llama3_8b_layer_shapes, numel, shard_numel, uneven_flat_numels

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    for opt in args.option:
        name, value = opt.split("=")
        _native.set_option(name, int(value))

    W = args.world_size
    shapes = llama3_8b_layer_shapes()
    if args.layout == "flat":
        shapes = [("flat", (sum(numel(s) for _, s in shapes),))]
    valid = [numel(s) for _, s in shapes]  # elements that exist; the rest of W * shard is padding
    if args.workload == "uneven":
        valid = uneven_flat_numels(40, W)
        shapes = [(f"flat{i}", (n,)) for i, n in enumerate(valid)]
    numels = [W * shard_numel(n, W) for n in valid]  # padded: what the kernels move
    padded = numels != valid
    assert padded == (args.workload == "uneven")
    N = sum(numels)
    per_rank = sum((n // W) * 6 + 512 for n in numels) + (1 << 20)
    group = odc_amd.init_nvshmem(world_size=W, symmetric_size=per_rank)
    registry = odc_amd.SymmBufferRegistry.get_instance()
    gather = odc_amd.GatherService()
    reduction = odc_amd.ReductionService(accumulation_dtype=torch.float32, lazy_clear=args.lazy_clear)

    # synthetic data, generated on the device and mirrored to the host for the oracle
    dev_gen = torch.Generator(device="cuda").manual_seed(0)
    params = [(torch.randn(n, generator=dev_gen, device="cuda") * 0.02).bfloat16() for n in numels]
    for p, v in zip(params, valid):
        p[v:] = 0  # the zero padding of the last shards (odc/fsdp/fsdp1.py:239-247)
    grads = [[(torch.randn(v, generator=dev_gen, device="cuda") * 1e-3).bfloat16() for v in valid]
             for _ in range(MICROBATCHES)]
    keys = [name for name, _ in shapes]
    shard_locals = []
    for key, p in zip(keys, params):
        for r in range(W):
            with odc_amd.virtual_rank(r):
                t = registry.update_symm_buffer(key, p.view(W, -1)[r])
        shard_locals.append(registry.get_symm_buffer(key))
    outs = [torch.empty_like(p) for p in params]
    # register the accumulations up front (lazy registration is not part of a steady-state step)
    for key, n in zip(keys, numels):
        reduction.register(key, (n // W,), torch.bfloat16, torch.float32, group)
    torch.cuda.synchronize()

    comm = get_comm_stream()
    # One event after every launch of the timed region (plus one at its start): launch k's
    # duration is the time between marks k and k+1, all recorded on the launch stream.
    marks = []

    def mark(label):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(comm)
        marks.append((label, ev))

    def step(i, record):
        m = i % MICROBATCHES
        if m == 0:
            reduction.clear_accumulations()
            if record and not args.lazy_clear:
                mark("clear")
        gather.gather_into_tensors(outs, shard_locals, group)
        if record:
            mark("gather")
        reduction.scatter_accumulate_multi(keys, grads[m], group, valid_numels=valid if padded else None)
        if record:
            mark("store" if m == 0 and args.lazy_clear else "accum")

    # ---- parity + CPU baseline: one full minibatch against the oracle -------------------------
    cpu_baseline = None
    parity = None
    if not args.no_verify or not args.no_cpu_baseline:
        from oracle import odc_oracle as oracle

        for i in range(MICROBATCHES):
            step(i, record=False)
        reduction.sync(group)
        host_params = [p.cpu() for p in params]
        host_grads = [[torch.cat([g.cpu(), torch.zeros(n - g.numel(), dtype=g.dtype)]) if padded else g.cpu()
                       for g, n in zip(mb, numels)] for mb in grads]
        host_outs = [torch.empty_like(p) for p in host_params]
        host_accs = [[torch.zeros(n // W, dtype=torch.float32) for _ in range(W)] for n in numels]
        host_shards = [list(p.view(W, -1)) for p in host_params]
        def cpu_minibatch():
            for m in range(MICROBATCHES):
                for o, sh in zip(host_outs, host_shards):
                    oracle.gather_into_tensor(o, sh)
                for accs, g in zip(host_accs, host_grads[m]):
                    oracle.scatter_accumulate(accs, g)

        t0 = time.perf_counter()
        cpu_minibatch()  # this first pass also produces the values the GPU is checked against
        first_s = time.perf_counter() - t0
        check_accs = [[a.clone() for a in accs] for accs in host_accs]
        cpu_s, passes = first_s, 1
        if not args.no_cpu_baseline:
            while cpu_s < args.cpu_seconds:  # bounded sample: about 10 s of CPU work
                t0 = time.perf_counter()
                cpu_minibatch()
                cpu_s += time.perf_counter() - t0
                passes += 1
        host_accs = check_accs
        cpu_baseline = {
            "value": round(passes * MICROBATCHES * 14 * N / cpu_s / 1e9, 3),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{passes} x {MICROBATCHES} microbatches of the same layer (gather + "
                      f"scatter-accumulate) through the torch CPU oracle, {cpu_s:.1f} s",
        }
        if args.no_cpu_baseline:
            cpu_baseline = None
        if not args.no_verify:
            ok = True
            for o, ho in zip(outs, host_outs):
                ok &= torch.equal(o.cpu().view(torch.int16), ho.view(torch.int16))
            for key, accs in zip(keys, host_accs):
                for r, acc in enumerate(reduction.get_peer_accumulations(key)):
                    ok &= torch.equal(acc.cpu().view(torch.int32), accs[r].view(torch.int32))
            parity = bool(ok)
            if not ok:
                print("PARITY FAILURE: GPU results differ from the CPU oracle", file=sys.stderr)
        del host_params, host_grads, host_outs, host_accs, host_shards

    # ---- timed region -----------------------------------------------------------------------
    # The services launch on the caller's current stream. The timed loop runs on a side stream
    # of its own (not torch's default stream), and the events are recorded on that same stream,
    # so that each pair of events brackets exactly one kernel.
    # A full Python garbage collection (tens of ms with torch imported) landing inside the timed
    # loop would stall the launches while an event pair is open: collect now, then keep the
    # collector off until the loop is done.
    gc.collect()
    gc.disable()
    with torch.cuda.stream(comm):
        for i in range(args.warmup):
            step(i, record=False)
        torch.cuda.synchronize()
        host_step = []
        mark("start")
        t0 = time.perf_counter()
        for i in range(args.steps):
            ts = time.perf_counter()
            step(i, record=True)
            host_step.append(time.perf_counter() - ts)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if os.environ.get("ODC_BENCH_DEBUG"):
            print("host ms per step:", [round(x * 1e3, 3) for x in host_step], file=sys.stderr)
        # the same steps once more in the other clear mode (no events): a secondary figure
        other = None
        if args.steps >= MICROBATCHES:
            reduction.lazy_clear = not args.lazy_clear
            for i in range(MICROBATCHES):
                step(i, record=False)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for i in range(args.steps):
                step(i, record=False)
            torch.cuda.synchronize()
            other_elapsed = time.perf_counter() - t1
            stores = len(range(0, args.steps, MICROBATCHES)) if reduction.lazy_clear else 0
            other_bytes = 14 * N * args.steps - 4 * N * stores
            other = {"clear": "lazy (store on the first microbatch)" if reduction.lazy_clear else "eager",
                     "value": round(other_bytes / other_elapsed / 1e9, 1), "unit": "GB/s",
                     "bytes_per_step": round(other_bytes / args.steps),
                     "minibatch_ms": round(other_elapsed / args.steps * MICROBATCHES * 1e3, 4)}
            reduction.lazy_clear = args.lazy_clear
    gc.enable()

    if args.calibrate:
        a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()

    durations = {"clear": [], "gather": [], "accum": [], "store": []}
    for (_, before), (label, after) in zip(marks, marks[1:]):
        durations[label].append(before.elapsed_time(after))

    def mean_ms(label):
        return statistics.fmean(durations[label]) if durations[label] else None

    def measured_traffic(kernel):
        return MEASURED_TRAFFIC_BYTES.get((kernel, args.layout, W)) if args.workload == "layer" else None

    g_ms, a_ms, c_ms, s_ms = mean_ms("gather"), mean_ms("accum"), mean_ms("clear"), mean_ms("store")
    if os.environ.get("ODC_BENCH_DEBUG"):
        print("gather ms per launch:", [round(x, 3) for x in durations["gather"]], file=sys.stderr)
        print("accum ms per launch:", [round(x, 3) for x in durations["accum"]], file=sys.stderr)
    accum_gbps = 10 * N / (a_ms * 1e-3) / 1e9
    gather_gbps = 4 * N / (g_ms * 1e-3) / 1e9
    # bytes the timed steps move by the algorithm: a store step's scatter moves 6N, not 10N
    step_bytes = (14 * N * args.steps - 4 * N * len(durations["store"])) / args.steps
    value = args.steps * step_bytes / elapsed / 1e9
    workload = (f"cfg2: Llama-3-8B decoder layer ({N} bf16 params, {len(keys)} tensors, "
                f"{args.layout}), W={W} virtual shards, {MICROBATCHES} microbatches per minibatch")
    if args.workload == "uneven":
        workload = (f"cfg3: {len(keys)} flat bf16 parameters of log-uniform size ({sum(valid)} elements, "
                    f"{N} with the zero padding of the shards), none divisible by W={W}, "
                    f"{MICROBATCHES} microbatches per minibatch")
    result = {
        "metric": "achieved HBM GB/s (% of ~8 TB/s peak) for gather + scatter-accum, 8B layer, W=8",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": workload, "world_size": W, "elements": N,
                   "bytes_per_step": round(step_bytes), "layout": args.layout,
                   "clear": "lazy (store on the first microbatch)" if args.lazy_clear else "eager"},
        "frac_of_peak": round(value / HBM_PEAK_GBPS, 4),
        "roofline": {
            "kernel": "accum_kernel<bf16,f32> (scatter-accumulate)",
            "bound": "hbm",
            "achieved": round(accum_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(accum_gbps / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("accum"),
            "algorithmic_bytes": 10 * N,
            "avg_launch_ms": round(a_ms, 5),
            "min_launch_ms": round(min(durations["accum"]), 5),
            "max_launch_ms": round(max(durations["accum"]), 5),
        },
        "roofline_gather": {
            "kernel": "gather_kernel",
            "bound": "hbm",
            "achieved": round(gather_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(gather_gbps / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic("gather"),
            "algorithmic_bytes": 4 * N,
            "avg_launch_ms": round(g_ms, 5),
            "min_launch_ms": round(min(durations["gather"]), 5),
            "max_launch_ms": round(max(durations["gather"]), 5),
        },
        "clear": {"avg_launch_ms": round(c_ms, 5) if c_ms else None,
                  "GB/s": round(4 * N / (c_ms * 1e-3) / 1e9, 1) if c_ms else None},
        "store": {"avg_launch_ms": round(s_ms, 5) if s_ms else None,
                  "GB/s": round(6 * N / (s_ms * 1e-3) / 1e9, 1) if s_ms else None,
                  "traffic": measured_traffic("store") if s_ms else None},
        "minibatch_ms": round(elapsed / args.steps * MICROBATCHES * 1e3, 4),
        "other_clear_mode": other,
        "cpu_baseline": cpu_baseline,
        "parity_vs_oracle": parity,
    }
    print(json.dumps(result))
    torch.cuda.synchronize()
    registry.finalize()
    odc_amd.finalize_distributed()
    if parity is False:
        sys.exit(1)


if __name__ == "__main__":
    main()
