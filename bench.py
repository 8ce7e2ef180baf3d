#!/usr/bin/env python3
"""Benchmark of the ODC hot path on one MI355X: gather + scatter-accumulate over a Llama-3-8B
decoder layer sharded over W=8 virtual ranks.

One step = one microbatch of the path over the whole layer:
    gather            all 9 parameters, bf16, W shards -> full tensors      (one launch, 4N bytes)
    scatter-accumulate all 9 bf16 gradients into the W fp32 accumulations   (one launch, 10N bytes)
Every 8th step starts a new minibatch and first clears the accumulations (inside the timed
region; its 4N written bytes are NOT counted in the numerator).

The headline (`value`, `ms_per_step`) times EXACTLY --steps steps replayed from HIP graphs: one
graph per whole minibatch (clear + 8 x (gather + scatter-accumulate)), one more for the steps left
over; `--no-graph` launches them eagerly instead. After that, a short eager phase records one HIP
event on the launch stream after every launch: per-kernel durations for `roofline` (the
scatter-accumulate, the dominant kernel) and `roofline_gather`.

Prints ONE JSON line with, besides the contract's fields: `roofline.practical_ceiling` (what bare
streaming kernels of libodc_ceiling.so reach on flat arrays of the same sizes in the same run),
`roofline.traffic` (HBM bytes per launch from the committed rocprofv3 counter runs listed in
profiles/traffic.json; null when a launch knob is overridden), `host_us_per_call` (host time of one
call of each service entry point on the 9-parameter layer), the clear, the CPU oracle timed on
the host cores (`cpu_baseline`), the parity verdict against that oracle, and `other_clear_mode`:
the same minibatches with lazy clears, replayed from a graph captured inside
`ReductionService.captured_minibatch()`: no clear kernel runs and the first scatter-accumulate of
a minibatch stores instead (6N bytes, counted as such), checked against the oracle as well.

Other workloads (not the headline): `--workload uneven --world-size 12` (40 uneven, zero-padded
flat parameters), `--workload model` (the whole 8.03 G-parameter model, swept unit by unit: sampled
units against the oracle, per-unit-shape roofline figures, a CPU baseline extrapolated from the
embedding and one layer), `--layout flat`, `--world-size 64`.
"""

from __future__ import annotations

import argparse
import ctypes
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
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"


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
    ap.add_argument("--no-graph", action="store_true",
                    help="launch the timed steps eagerly instead of replaying HIP graphs")
    ap.add_argument("--event-steps", type=int, default=104,
                    help="eager steps with one HIP event per launch, for the per-kernel roofline figures")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the bare streaming kernels")
    ap.add_argument("--no-host-overhead", action="store_true", help="skip the host-time-per-call measurement")
    ap.add_argument("--no-launch-floor", action="store_true",
                    help="skip the one-tile launches (they would skew a profiler's per-kernel averages)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="CPU baseline sample length")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--lazy-clear", action="store_true",
                    help="lazy clears for the headline: no clear kernel, the first scatter-accumulate of a "
                         "minibatch stores instead (6N bytes); graphs are then captured inside "
                         "captured_minibatch(). The default keeps the reference's eager clears, so that every "
                         "timed scatter-accumulate is the 10N read-modify-write")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one torch copy of 1 GiB (counter calibration under rocprofv3)")
    ap.add_argument("--probe", choices=["alignment", "overlap", "tiny-items"],
                    help="instead of the benchmark, print one of three measurement tables: alignment (what a buffer "
                         "shifted off the 16 KiB tile grid costs the scatter-accumulate and the gather), overlap (how "
                         "much of a gather / scatter-accumulate hides behind a co-running GEMM, by launch shape), "
                         "tiny-items (what items of less than one tile per rank cost the scatter-accumulate by their "
                         "place in the launch order; run it with --world-size 64)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="libodc_hip launch knob, e.g. accum_blocks_per_cu=4")
    return ap.parse_args()


def model_sweep(args):
    """Full Llama-3-8B (cfg 5): per step (= microbatch), gather the 34 FSDP units in forward order,
    then scatter-accumulate them in reverse order; every 8th step first clears all accumulations.

    Parity: one eager minibatch, then the sampled units (embedding, two layers, head) against the
    CPU oracle, gather and all W accumulations, bit for bit. CPU baseline: the oracle timed on the
    embedding and one layer (a ninth of the model's bytes) and extrapolated to the sweep. Roofline:
    an eager event phase with one HIP event after every launch, reported for the scatter-accumulate
    over the whole sweep and per unit shape."""
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
    shape_of = ["embedding"] + ["layer"] * (len(units) - 2) + ["head"]
    unit_elems = [sum(numel(s) for _, s in unit) for _, unit in units]
    marks = []

    def mark(label):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(comm)
        marks.append((label, ev))

    def step(i, record=False):
        if i % MICROBATCHES == 0:
            reduction.clear_accumulations()
            if record and not reduction.lazy_clear:
                mark(("clear", "all"))
        for u, (keys, locals_, outs, grads) in enumerate(plan):
            gather.gather_into_tensors(outs, locals_, group)
            if record:
                mark(("gather", shape_of[u]))
        store = reduction.lazy_clear and i % MICROBATCHES == 0
        for u in reversed(range(len(plan))):
            keys, locals_, outs, grads = plan[u]
            reduction.scatter_accumulate_multi(keys, grads[i % 2], group)
            if record:
                mark(("store" if store else "accum", shape_of[u]))

    # ---- parity + CPU baseline on sampled units -------------------------------------------------
    parity = cpu_baseline = None
    if not args.no_verify or not args.no_cpu_baseline:
        from oracle import odc_oracle as oracle

        with torch.cuda.stream(comm):
            for i in range(MICROBATCHES):
                step(i)
        reduction.sync(group)
        sampled = [0, 1, len(units) // 2, len(units) - 1]  # embedding, two layers, norm + lm_head
        timed_units = {0, 1}  # the CPU baseline's sample: the embedding and one layer
        parity = True
        cpu_s = cpu_bytes = 0.0
        cpu_passes = 0
        for u in sampled:
            keys, locals_, outs, grads = plan[u]
            host_shards = [[peer.cpu() for peer in registry.peer_tensors[k]] for k in keys]
            host_grads = [[g.cpu() for g in mb] for mb in grads]
            host_outs = [torch.empty(o.numel(), dtype=torch.bfloat16) for o in outs]
            host_accs = [[torch.zeros(o.numel() // W) for _ in range(W)] for o in outs]

            def cpu_minibatch():
                for m in range(MICROBATCHES):
                    for o, sh in zip(host_outs, host_shards):
                        oracle.gather_into_tensor(o, sh)
                    for accs, g in zip(host_accs, host_grads[m % 2]):
                        oracle.scatter_accumulate(accs, g)

            t0 = time.perf_counter()
            cpu_minibatch()  # the values the GPU is checked against
            first_s = time.perf_counter() - t0
            if not args.no_verify:
                with torch.cuda.stream(comm):
                    gather.gather_into_tensors(outs, locals_, group)  # the buffers are shared by shape: gather again
                torch.cuda.synchronize()
                for o, ho in zip(outs, host_outs):
                    parity &= torch.equal(o.cpu().view(torch.int16), ho.view(torch.int16))
                for key, accs in zip(keys, host_accs):
                    for r, acc in enumerate(reduction.get_peer_accumulations(key)):
                        parity &= torch.equal(acc.cpu().view(torch.int32), accs[r].view(torch.int32))
            if u in timed_units and not args.no_cpu_baseline:
                budget = args.cpu_seconds * unit_elems[u] / sum(unit_elems[t] for t in timed_units)
                spent, passes = first_s, 1
                while spent < budget:
                    t0 = time.perf_counter()
                    cpu_minibatch()
                    spent += time.perf_counter() - t0
                    passes += 1
                cpu_s += spent
                cpu_bytes += passes * MICROBATCHES * 14 * unit_elems[u]
                cpu_passes += passes
            del host_shards, host_grads, host_outs, host_accs
        parity = bool(parity) if not args.no_verify else None
        if parity is False:
            print("PARITY FAILURE: GPU results differ from the CPU oracle on a sampled unit", file=sys.stderr)
        if not args.no_cpu_baseline:
            rate = cpu_bytes / cpu_s / 1e9
            cpu_baseline = {
                "value": round(rate, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": f"{cpu_passes} minibatches of {MICROBATCHES} microbatches over the embedding and one decoder "
                          f"layer ({sum(unit_elems[t] for t in timed_units)} of {N} elements) through the torch CPU "
                          f"oracle, {cpu_s:.1f} s; EXTRAPOLATED to the sweep at that rate: "
                          f"{14 * N / rate / 1e9:.2f} s per microbatch",
            }

    # ---- headline: exactly --steps steps, eager launches ------------------------------------------
    gc.collect()
    gc.disable()
    with torch.cuda.stream(comm):
        for i in range(-(-args.warmup // MICROBATCHES) * MICROBATCHES):
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
        # ---- eager event phase: one event after every launch --------------------------------------
        mark(("start", ""))
        for i in range(MICROBATCHES if args.event_steps > 0 else 0):  # one minibatch: 544 launches
            step(i, record=True)
        torch.cuda.synchronize()
    gc.enable()
    if args.calibrate:
        a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()

    durations = {}
    for (_, before), (label, after) in zip(marks, marks[1:]):
        durations.setdefault(label, []).append(before.elapsed_time(after))
    shape_elems = {"embedding": unit_elems[0], "layer": unit_elems[1], "head": unit_elems[-1]}
    traffic = load_traffic(args, W)

    def kernel_figures(kind, bytes_per_elem):
        """Per unit shape and over the whole sweep: mean launch time, GB/s, fraction of peak."""
        per_shape, total_bytes, total_ms = {}, 0.0, 0.0
        for shape, elems in shape_elems.items():
            times = durations.get((kind, shape))
            if not times:
                continue
            ms = statistics.fmean(times)
            gbps = bytes_per_elem * elems / (ms * 1e-3) / 1e9
            per_shape[shape] = {"elements": elems, "avg_launch_ms": round(ms, 5), "launches_timed": len(times),
                                "GB/s": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
            total_bytes += bytes_per_elem * elems * len(times)
            total_ms += sum(times)
        if not per_shape:
            return None, None, None
        return per_shape, total_bytes, total_ms

    roofline = roofline_gather = None
    accum_shapes, accum_bytes, accum_ms = kernel_figures("accum", 10)
    if accum_shapes:
        launches = sum(v["launches_timed"] for v in accum_shapes.values())
        gbps = accum_bytes / (accum_ms * 1e-3) / 1e9
        entry = traffic.get("accum:embedding", (None, None))
        roofline = {
            "kernel": "accum_kernel<bf16,f32> (scatter-accumulate), all launches of the sweep",
            "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes": round(accum_bytes / launches), "avg_launch_ms": round(accum_ms / launches, 5),
            "launches_timed": launches,
            "traffic": entry[0], "traffic_source": entry[1],
            "traffic_launch": "the embedding-sized launch (algorithmic bytes "
                              f"{10 * shape_elems['embedding']})" if entry[0] else None,
            "by_unit_shape": accum_shapes,
        }
    gather_shapes, gather_bytes, gather_ms = kernel_figures("gather", 4)
    if gather_shapes:
        launches = sum(v["launches_timed"] for v in gather_shapes.values())
        gbps = gather_bytes / (gather_ms * 1e-3) / 1e9
        entry = traffic.get("gather:embedding", (None, None))
        roofline_gather = {
            "kernel": "gather_kernel, all launches of the sweep", "bound": "hbm", "achieved": round(gbps, 1),
            "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes": round(gather_bytes / launches), "avg_launch_ms": round(gather_ms / launches, 5),
            "launches_timed": launches, "traffic": entry[0], "traffic_source": entry[1],
            "by_unit_shape": gather_shapes,
        }
    store_shapes, _, _ = kernel_figures("store", 6)
    clear_ms = statistics.fmean(durations[("clear", "all")]) if durations.get(("clear", "all")) else None

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
                   "bytes_per_step": round(step_bytes), "launch": "eager",
                   "clear": "lazy (store on the first microbatch)" if args.lazy_clear else "eager"},
        "minibatch_ms": round(elapsed / args.steps * MICROBATCHES * 1e3, 3),
        "frac_of_peak": round(value / HBM_PEAK_GBPS, 4),
        "gpu_ms_per_step": round(e0.elapsed_time(e1) / args.steps, 3),
        "roofline": roofline, "roofline_gather": roofline_gather,
        "store": store_shapes,
        "clear": {"avg_launch_ms": round(clear_ms, 4), "GB/s": round(4 * N / (clear_ms * 1e-3) / 1e9, 1)} if clear_ms else None,
        "cpu_baseline": cpu_baseline, "parity_vs_oracle": parity,
        "parity_sample": "units 0 (embedding), 1 and 17 (decoder layers), 33 (final norm + lm_head): gathered "
                         "parameters and all W accumulations after one minibatch, bit for bit",
    }))
    torch.cuda.synchronize()
    registry.finalize()
    odc_amd.finalize_distributed()
    if parity is False:
        sys.exit(1)


def load_traffic(args, W):
    """HBM bytes per launch from the committed rocprofv3 counter runs: kernel -> (bytes, source).
    Only for the configuration those runs profiled, and only with the library's default knobs."""
    if args.option or not TRAFFIC_FILE.exists():
        return {}
    try:
        table = json.loads(TRAFFIC_FILE.read_text())
    except (OSError, ValueError):
        return {}
    out = {}
    for e in table.get("entries", []):
        if (e.get("workload"), e.get("layout"), e.get("world_size")) == (args.workload, args.layout, W):
            # the model sweep launches one kernel at several sizes: its entries name the unit shape
            name = e["kernel"] + (":" + e["unit_shape"] if e.get("unit_shape") else "")
            out[name] = (e["hbm_bytes_per_launch"],
                         f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, {e['profile']} (not measured by this run)")
    return out


def measure_ceiling(torch, comm, N, iters=12):
    """Bare streaming kernels over flat arrays of the layer's sizes, launched alternately (copy,
    read-modify-write, read, write: every launch meets cold caches, as the real steps do) with
    one HIP event after each. Four launch shapes each; the best average is the ceiling."""
    from odc_amd import _native

    lib = _native.load_ceiling()
    # every kernel has arrays of its own: what one leaves in the 256 MB last-level cache must not
    # be what the next one reads (a write pass over the accumulation would hand the following
    # read-modify-write a quarter of its accumulation reads from cache)
    src = torch.empty(N, dtype=torch.bfloat16, device="cuda").normal_(0, 0.02)
    dst = torch.empty_like(src)
    grad = torch.empty(N, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3)
    acc = torch.zeros(N, dtype=torch.float32, device="cuda")
    read_only = torch.zeros(N, dtype=torch.float32, device="cuda")
    write_only = torch.empty(N, dtype=torch.float32, device="cuda")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(comm.cuda_stream)
    moved = ctypes.c_uint64()
    # (persistent workgroups per CU or 0, unused LDS claimed per workgroup, threads per workgroup)
    shapes = {"one workgroup per tile": (0, 0, 256), "one per tile, 4 resident per CU": (0, 40960, 256),
              "1 persistent workgroup per CU": (1, 0, 256), "one 512-thread workgroup per tile": (0, 0, 512)}

    def launch(kind, wg, lds):
        if kind == "copy":
            rc = lib.odc_ceiling_copy(dst.data_ptr(), src.data_ptr(), 2 * N, wg, lds, stream, ctypes.byref(moved))
        elif kind == "rmw_bf16_f32":
            rc = lib.odc_ceiling_rmw(acc.data_ptr(), grad.data_ptr(), N, wg, lds, stream, ctypes.byref(moved))
        elif kind == "read":
            rc = lib.odc_ceiling_read(read_only.data_ptr(), 4 * N, sink.data_ptr(), wg, lds, stream, ctypes.byref(moved))
        else:
            rc = lib.odc_ceiling_write(write_only.data_ptr(), 4 * N, wg, lds, stream, ctypes.byref(moved))
        assert rc == 0, f"ceiling kernel {kind} failed to launch"
        return moved.value

    kinds = ("copy", "rmw_bf16_f32", "read", "write")
    table = {k: {} for k in kinds}
    with torch.cuda.stream(comm):
        for label, (wg, lds, threads) in shapes.items():
            assert lib.odc_ceiling_set_threads(threads) == 0
            marks, nbytes = [], {}
            for it in range(iters + 2):
                for kind in kinds:
                    e0 = torch.cuda.Event(enable_timing=True)
                    e0.record(comm)
                    nbytes[kind] = launch(kind, wg, lds)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e1.record(comm)
                    if it >= 2:
                        marks.append((kind, e0, e1))
            torch.cuda.synchronize()
            for kind in kinds:
                ms = statistics.fmean(a.elapsed_time(b) for k, a, b in marks if k == kind)
                table[kind][label] = round(nbytes[kind] / (ms * 1e-3) / 1e9, 1)
    best = {k: max(v.values()) for k, v in table.items()}
    return {"unit": "GB/s", **best, "by_launch_shape": table,
            "note": "bare kernels of libodc_ceiling.so on flat arrays of the layer's sizes (copy 2 x 2N bytes, "
                    "rmw 10N, read 4N, write 4N; separate arrays per kernel), launched alternately, HIP events "
                    "per launch"}


def measure_launch_floor(torch, comm, group, gather, reduction, registry, W, launches=50):
    """What a launch costs before any bandwidth: gather and scatter-accumulate of ONE 64-element
    item (one 128-byte slice per rank, the smallest shard of the layer at W=64), event to event on
    the launch stream, and the same with the device idle before each launch."""
    small = registry.allocate_symm_buffer("bench_floor_shard", (64,), torch.bfloat16)
    out = torch.empty(W * 64, dtype=torch.bfloat16, device="cuda")
    grad = torch.zeros(W * 64, dtype=torch.bfloat16, device="cuda")
    reduction.register("bench_floor", (64,), torch.bfloat16, torch.float32, group)
    torch.cuda.synchronize()
    result = {}
    with torch.cuda.stream(comm):
        for label, fn in (("gather_one_tile", lambda: gather.gather_into_tensor(out, small, group)),
                          ("scatter_accumulate_one_tile", lambda: reduction.scatter_accumulate("bench_floor", grad, group))):
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            events = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
            events[0].record(comm)
            for k in range(launches):
                fn()
                events[k + 1].record(comm)
            torch.cuda.synchronize()
            back_to_back = statistics.fmean(a.elapsed_time(b) for a, b in zip(events, events[1:])) * 1e3
            idle = []
            for _ in range(launches):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(comm)
                fn()
                e1.record(comm)
                torch.cuda.synchronize()
                idle.append(e0.elapsed_time(e1) * 1e3)
            # the same launches replayed from one HIP graph: no host time between them
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(launches):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g0.record(comm)
            graph.replay()
            g1.record(comm)
            torch.cuda.synchronize()
            result[label] = {"eager_back_to_back_us": round(back_to_back, 2),
                             "eager_from_idle_us": round(statistics.median(idle), 2),
                             "graph_replay_us": round(g0.elapsed_time(g1) * 1e3 / launches, 2)}
            del graph
    result["note"] = (f"microseconds per launch of one 64-element item (W x 128 B): HIP-event interval, mean of "
                      f"{launches} eager launches queued back to back (bounded by the host's time per call), "
                      "median when the device is idle before each, and per launch when the same "
                      f"{launches} launches are replayed from one HIP graph (the device-side floor)")
    return result


def measure_host_overhead(torch, odc_amd, comm, group, gather, reduction, registry, outs, shard_locals, keys,
                          grads, numels, W, calls=100):
    """Host time of one call, mean over `calls` back-to-back asynchronous calls (the launches
    queue up; the device is drained afterwards): the multi-tensor entry points on the 9 tensors,
    and the slice entry points (the FSDP2 group path) on the same layer as one group buffer."""
    result = {}

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            fn()
        dt = time.perf_counter() - t0
        torch.cuda.synchronize()
        return round(dt / calls * 1e6, 2)

    with torch.cuda.stream(comm):
        n = len(keys)
        result[f"gather_into_tensors[{n}]"] = timed(lambda: gather.gather_into_tensors(outs, shard_locals, group))
        result[f"scatter_accumulate_multi[{n}]"] = timed(
            lambda: reduction.scatter_accumulate_multi(keys, grads, group))
        shard_numels = [x // W for x in numels]
        offsets = [0]
        for s in shard_numels:
            offsets.append(offsets[-1] + s)
        total = offsets.pop()
        group_buffer = registry.allocate_symm_buffer("bench_group_buffer", (total,), torch.bfloat16)
        result[f"gather_slices[{n}]"] = timed(
            lambda: gather.gather_slices(outs, group_buffer, offsets, shard_numels, group))
        result[f"scatter_accumulate_slices[{n}]"] = timed(
            lambda: reduction.scatter_accumulate_slices("bench_group", grads, offsets, shard_numels, group,
                                                        accumulation_numel=total))
    result["note"] = f"host microseconds per call, mean of {calls} asynchronous calls"
    return result


def probe_alignment(args, repeats=9, launches=20):
    """`--probe alignment`: what a misaligned buffer costs the streaming kernels. One
    scatter-accumulate (bf16 into fp32, read-modify-write) and one gather of a buffer too large for
    the last-level cache, with the accumulation slice, the gradient, the shard slice and the output
    each shifted by 0 ... 16 KiB. (On MI355X the read-modify-write loses up to 5.5 % when its tiles
    start 8 KiB past a 16 KiB boundary of the ACCUMULATION and nothing when the gradient is shifted,
    the gather about 1 % per shifted side: why the arena and the FSDP2 group layout start buffers
    and slices on tile boundaries.) Median of `repeats` intervals of `launches` launches."""
    import torch

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
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(launches):
                fn()
            e1.record()
            e1.synchronize()
            samples.append(e0.elapsed_time(e1) / launches)
        return statistics.median(samples)

    shifts = (0, 2048, 4096, 8192, 12288, 16384)
    outside = torch.empty(W * n_gat * 2 + (1 << 20), dtype=torch.uint8, device="cuda")  # gradient, then output
    outside.view(torch.bfloat16).normal_(0, 1e-3)
    reduction.register("acc", (n_acc + slack,), torch.bfloat16, torch.float32, group)
    print(f"scatter-accumulate, {W} x {n_acc} elements, GB/s by byte shift of the slice in the accumulation (rows) "
          f"and of the gradient (columns)")
    print(f"{'':>8s}" + "".join(f"{g:>8d}" for g in shifts))
    for a in shifts:
        row = []
        for g in shifts:
            grad = outside[g:g + W * n_acc * 2].view(torch.bfloat16)
            ms = timed(lambda: reduction.scatter_accumulate_slices("acc", [grad], [a // 4], [n_acc], group))
            row.append(10 * W * n_acc / ms / 1e6)
        print(f"{a:>8d}" + "".join(f"{x:8.0f}" for x in row), flush=True)
    shards = registry.allocate_symm_buffer("shards", (n_gat + slack,), torch.bfloat16)
    print(f"gather, {W} x {n_gat} bf16 elements, GB/s by byte shift of the shard slice (rows) and of the output (columns)")
    print(f"{'':>8s}" + "".join(f"{d:>8d}" for d in shifts))
    for sh in shifts:
        row = []
        for d in shifts:
            out = outside[d:d + W * n_gat * 2].view(torch.bfloat16)
            ms = timed(lambda: gather.gather_slices([out], shards, [sh // 2], [n_gat], group))
            row.append(4 * W * n_gat / ms / 1e6)
        print(f"{sh:>8d}" + "".join(f"{x:8.0f}" for x in row), flush=True)
    torch.cuda.synchronize()
    registry.finalize()
    odc.finalize_distributed()


def probe_tiny_items(args, launches=40):
    """`--probe tiny-items`: the 9-parameter layer's scatter-accumulate, launched back to back, with
    its two norm items (64 elements per rank at W=64: less than one tile) where the caller lists
    them (between the projection matrices), launched last (the library's default), and left out;
    one workgroup per tile and one persistent workgroup per CU; rank-outermost and item-major."""
    import torch

    import odc_amd as odc
    from odc_amd import _native
    from odc_amd.workloads import llama3_8b_layer_shapes, numel

    W = args.world_size
    torch.cuda.set_device(0)
    shapes = llama3_8b_layer_shapes()
    numels = {name: numel(s) for name, s in shapes}
    group = odc.init_nvshmem(world_size=W, symmetric_size=sum(v // W * 4 + 32768 for v in numels.values()) + (8 << 20))
    reduction = odc.ReductionService(accumulation_dtype=torch.float32)
    grads = {name: torch.empty(v, dtype=torch.bfloat16, device="cuda").normal_(0, 1e-3) for name, v in numels.items()}
    for name, v in numels.items():
        reduction.register(name, (v // W,), torch.bfloat16, torch.float32, group)
    lists = {"all 9 items": [name for name, _ in shapes],
             "without the norm items": [name for name, s in shapes if len(s) > 1]}

    def timed(keys):
        g = [grads[k] for k in keys]
        for _ in range(5):
            reduction.scatter_accumulate_multi(keys, g, group)
        torch.cuda.synchronize()
        events = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
        events[0].record()
        for i in range(launches):
            reduction.scatter_accumulate_multi(keys, g, group)
            events[i + 1].record()
        torch.cuda.synchronize()
        return statistics.fmean(a.elapsed_time(b) for a, b in zip(events, events[1:])) * 1e3

    print(f"scatter-accumulate of the Llama-3-8B layer, W={W}, microseconds per launch (mean of {launches} back to back)")
    print(f"{'items, launch order of the tiny ones':44s} {'tile order':16s} {'per tile':>9s} {'persistent':>11s}")
    try:
        for label, keys in lists.items():
            for last in ((0, 1) if len(keys) == 9 else (1,)):
                for order, order_name in ((2, "rank-outermost"), (1, "item-major")):
                    row = []
                    for blocks_per_cu in (0, 1):
                        _native.set_option("accum_small_items_last", last)
                        _native.set_option("accum_tile_order", order)
                        _native.set_option("accum_blocks_per_cu", blocks_per_cu)
                        row.append(timed(keys))
                    where = "" if len(keys) != 9 else (", tiny last" if last else ", as listed")
                    print(f"{label + where:44s} {order_name:16s} {row[0]:9.1f} {row[1]:11.1f}", flush=True)
    finally:
        _native.set_option("accum_small_items_last", 1)
        _native.set_option("accum_tile_order", 3)
        _native.set_option("accum_blocks_per_cu", -1)
    torch.cuda.synchronize()
    odc.SymmBufferRegistry.get_instance().finalize()
    odc.finalize_distributed()


def probe_overlap(args, gemm=8192, launches=8, repeats=5):
    """`--probe overlap`: how much of a gather / scatter-accumulate hides behind compute on ONE
    GPU. The reference hops to a side stream so that its data movement overlaps the model's compute
    (odc/primitives/gather.py:114-176, utils.py:205-209); there the movement crosses NVLink, here it
    is a streaming kernel that competes with the compute kernels for the same CUs and the same HBM.
    A chain of bf16 GEMMs (compute bound) on one stream, the layer's gather or scatter-accumulate
    launches on another, alone and together, by launch shape:
        hidden = (t_gemm + t_path - t_both) / t_path      1 = free, 0 = fully serialised"""
    import torch

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
    a = torch.randn(gemm, gemm, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(gemm, gemm, device="cuda", dtype=torch.bfloat16)
    c = torch.empty_like(a)
    compute, side = torch.cuda.Stream(), torch.cuda.Stream()

    def run_gather():
        for _ in range(launches):
            gather.gather_into_tensors(outs, shards, group)

    def run_accum():
        for _ in range(launches):
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
        return min(one(fn_side, n_gemm) for _ in range(repeats))

    t_gemm1 = best(None, 4) / 4
    print(f"bf16 GEMM {gemm}^3: {t_gemm1 * 1e3:.3f} ms = {2 * gemm ** 3 / t_gemm1 / 1e12:.0f} TFLOP/s; "
          f"layer of {N} elements, W={W}, {launches} launches per measurement")
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


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: W virtual ranks share one MI355X and nothing here uses a "
              "second GPU. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.probe:
        return {"alignment": probe_alignment, "overlap": probe_overlap, "tiny-items": probe_tiny_items}[args.probe](args)
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
    per_rank = sum((n // W) * 12 + 2048 for n in numels) + (2 << 20)  # shards, accumulations, and the same again as one group
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
                registry.update_symm_buffer(key, p.view(W, -1)[r])
        shard_locals.append(registry.get_symm_buffer(key))
    outs = [torch.empty_like(p) for p in params]
    # register the accumulations up front (lazy registration is not part of a steady-state step)
    for key, n in zip(keys, numels):
        reduction.register(key, (n // W,), torch.bfloat16, torch.float32, group)
    torch.cuda.synchronize()

    comm = get_comm_stream()
    # One event after every launch of the eager event phase (plus one at its start): launch k's
    # duration is the time between marks k and k+1, all recorded on the launch stream.
    marks = []

    def mark(label):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(comm)
        marks.append((label, ev))

    def step(i, record=False):
        m = i % MICROBATCHES
        if m == 0:
            reduction.clear_accumulations()
            if record and not reduction.lazy_clear:
                mark("clear")
        gather.gather_into_tensors(outs, shard_locals, group)
        if record:
            mark("gather")
        reduction.scatter_accumulate_multi(keys, grads[m], group, valid_numels=valid if padded else None)
        if record:
            mark("store" if m == 0 and reduction.lazy_clear else "accum")

    def check_against(host_outs, host_accs):
        ok = True
        for o, ho in zip(outs, host_outs):
            ok &= torch.equal(o.cpu().view(torch.int16), ho.view(torch.int16))
        for key, accs in zip(keys, host_accs):
            for r, acc in enumerate(reduction.get_peer_accumulations(key)):
                ok &= torch.equal(acc.cpu().view(torch.int32), accs[r].view(torch.int32))
        return bool(ok)

    # ---- parity + CPU baseline: one full minibatch against the oracle -------------------------
    cpu_baseline = None
    parity = None
    check_outs = check_accs = None
    if not args.no_verify or not args.no_cpu_baseline:
        from oracle import odc_oracle as oracle

        for i in range(MICROBATCHES):
            step(i)
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
        check_outs = host_outs
        cpu_s, passes = first_s, 1
        if not args.no_cpu_baseline:
            while cpu_s < args.cpu_seconds:  # bounded sample: about 10 s of CPU work
                t0 = time.perf_counter()
                cpu_minibatch()
                cpu_s += time.perf_counter() - t0
                passes += 1
            cpu_baseline = {
                "value": round(passes * MICROBATCHES * 14 * N / cpu_s / 1e9, 3),
                "unit": "GB/s",
                "cores": torch.get_num_threads(),
                "kind": "port",
                "sample": f"{passes} x {MICROBATCHES} microbatches of the same layer (gather + "
                          f"scatter-accumulate) through the torch CPU oracle, {cpu_s:.1f} s",
            }
        if not args.no_verify:
            parity = check_against(check_outs, check_accs)
            if not parity:
                print("PARITY FAILURE: GPU results differ from the CPU oracle (eager launches)", file=sys.stderr)
        del host_params, host_grads, host_accs, host_shards

    # ---- headline: exactly --steps steps -------------------------------------------------------
    # A full Python garbage collection (tens of ms with torch imported) landing inside a timed
    # loop would stall the launches: collect now, then keep the collector off until the end.
    gc.collect()
    gc.disable()
    full, rest = divmod(args.steps, MICROBATCHES)
    graph_mb = graph_rest = None

    def capture_steps(n):
        """One graph holding the first n steps of a minibatch (it starts with the clear). With lazy
        clears the capture runs inside captured_minibatch(): the captured clear records nothing and
        the first scatter-accumulate is recorded in the store form."""
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            if reduction.lazy_clear:
                with reduction.captured_minibatch():
                    for i in range(n):
                        step(i)
            else:
                for i in range(n):
                    step(i)
        return graph

    if not args.no_graph:
        # one graph per whole minibatch, one for the steps left over
        torch.cuda.synchronize()
        graph_mb = capture_steps(MICROBATCHES)
        if rest:
            graph_rest = capture_steps(rest)
        torch.cuda.synchronize()

    def run_steps(n_full, n_rest):
        if args.no_graph:
            for i in range(n_full * MICROBATCHES + n_rest):
                step(i)
        else:
            for _ in range(n_full):
                graph_mb.replay()
            if n_rest:
                graph_rest.replay()

    with torch.cuda.stream(comm):
        run_steps(-(-args.warmup // MICROBATCHES), 0)  # whole minibatches, at least --warmup steps
        if rest:
            run_steps(0, rest)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(full, rest)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if not args.no_graph and not args.no_verify and check_accs is not None:
            # the graphs must leave what the eager launches left: replay one minibatch and compare
            graph_mb.replay()
            torch.cuda.synchronize()
            graph_parity = check_against(check_outs, check_accs)
            if not graph_parity:
                print("PARITY FAILURE: graph replay differs from the CPU oracle", file=sys.stderr)
            parity = bool(parity and graph_parity)

        # ---- eager event phase: per-kernel durations ------------------------------------------
        graph_mb = graph_rest = None  # destroyed: nothing replays into the accumulations any more,
        reduction.forget_captured_graphs()  # so lazy clears may skip the clear kernel again
        for i in range(MICROBATCHES):
            step(i)
        torch.cuda.synchronize()
        mark("start")
        for i in range(max(args.event_steps, 1)):
            step(i, record=True)
        torch.cuda.synchronize()

        # the same steps once more in the other clear mode (no events): a secondary figure,
        # replayed from one graph per minibatch like the headline (capture_steps)
        other = None
        if args.steps >= MICROBATCHES:
            reduction.lazy_clear = not args.lazy_clear
            for i in range(MICROBATCHES):
                step(i)
            reduction.sync(group)
            other_parity = None
            if args.no_graph:
                t1 = time.perf_counter()
                for i in range(args.steps):
                    step(i)
                torch.cuda.synchronize()
                other_elapsed = time.perf_counter() - t1
                other_steps = args.steps
            else:
                other_graph = capture_steps(MICROBATCHES)
                other_graph.replay()
                torch.cuda.synchronize()
                t1 = time.perf_counter()
                for _ in range(max(full, 1)):
                    other_graph.replay()
                torch.cuda.synchronize()
                other_elapsed = time.perf_counter() - t1
                other_steps = max(full, 1) * MICROBATCHES
                if not args.no_verify and check_accs is not None:
                    other_parity = check_against(check_outs, check_accs)
                    if not other_parity:
                        print("PARITY FAILURE: the captured minibatch with the clear folded into a store differs "
                              "from the CPU oracle", file=sys.stderr)
                    parity = bool(parity and other_parity)
                del other_graph
                reduction.forget_captured_graphs()
            stores = len(range(0, other_steps, MICROBATCHES)) if reduction.lazy_clear else 0
            other_bytes = 14 * N * other_steps - 4 * N * stores
            other = {"clear": "lazy (store on the first microbatch)" if reduction.lazy_clear else "eager",
                     "launch": "eager" if args.no_graph else
                               f"HIP graph replay ({max(full, 1)} x one minibatch of {MICROBATCHES} steps"
                               + (", clear folded into the first scatter-accumulate)" if reduction.lazy_clear else ")"),
                     "value": round(other_bytes / other_elapsed / 1e9, 1), "unit": "GB/s",
                     "frac_of_peak": round(other_bytes / other_elapsed / 1e9 / HBM_PEAK_GBPS, 4),
                     "bytes_per_step": round(other_bytes / other_steps), "steps": other_steps,
                     "minibatch_ms": round(other_elapsed / other_steps * MICROBATCHES * 1e3, 4),
                     "parity_vs_oracle": other_parity}
            reduction.lazy_clear = args.lazy_clear
            reduction.clear_accumulations()
            reduction.sync(group)

    host_overhead = None
    if not args.no_host_overhead and not padded:
        host_overhead = measure_host_overhead(torch, odc_amd, comm, group, gather, reduction, registry, outs,
                                              shard_locals, keys, grads[0], numels, W)
    launch_floor = None
    if not args.no_launch_floor:
        launch_floor = measure_launch_floor(torch, comm, group, gather, reduction, registry, W)
    ceiling = None
    if not args.no_ceiling:
        ceiling = measure_ceiling(torch, comm, N)
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

    traffic = load_traffic(args, W)
    g_ms, a_ms, c_ms, s_ms = mean_ms("gather"), mean_ms("accum"), mean_ms("clear"), mean_ms("store")
    accum_gbps = 10 * N / (a_ms * 1e-3) / 1e9
    gather_gbps = 4 * N / (g_ms * 1e-3) / 1e9
    # bytes the timed steps move by the algorithm: a store step's scatter moves 6N, not 10N
    timed_stores = len(range(0, args.steps, MICROBATCHES)) if args.lazy_clear else 0
    step_bytes = (14 * N * args.steps - 4 * N * timed_stores) / args.steps
    value = args.steps * step_bytes / elapsed / 1e9
    clears = 0 if args.lazy_clear else full + (1 if rest else 0)
    kernel_sum_ms = None
    if c_ms is not None or args.lazy_clear:
        accum_like = a_ms * (args.steps - timed_stores) + (s_ms or 0.0) * timed_stores
        kernel_sum_ms = (g_ms * args.steps + accum_like + (c_ms or 0.0) * clears) / args.steps
    workload = (f"cfg2: Llama-3-8B decoder layer ({N} bf16 params, {len(keys)} tensors, "
                f"{args.layout}), W={W} virtual shards, {MICROBATCHES} microbatches per minibatch")
    if args.workload == "uneven":
        workload = (f"cfg3: {len(keys)} flat bf16 parameters of log-uniform size ({sum(valid)} elements, "
                    f"{N} with the zero padding of the shards), none divisible by W={W}, "
                    f"{MICROBATCHES} microbatches per minibatch")
    if ceiling is not None:
        ceiling = dict(ceiling)
        ceiling["accum_frac_of_rmw_ceiling"] = round(accum_gbps / ceiling["rmw_bf16_f32"], 4)
        ceiling["gather_frac_of_copy_ceiling"] = round(gather_gbps / ceiling["copy"], 4)
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
                   "clear": "lazy (store on the first microbatch)" if args.lazy_clear else "eager",
                   "launch": "eager" if args.no_graph else
                             f"HIP graph replay ({full} x one minibatch of {MICROBATCHES} steps"
                             + (f" + one graph of {rest} steps)" if rest else ")"),
                   "clears_in_timed_region": clears},
        "frac_of_peak": round(value / HBM_PEAK_GBPS, 4),
        "kernel_sum_ms_per_step": round(kernel_sum_ms, 4) if kernel_sum_ms else None,
        "roofline": {
            "kernel": "accum_kernel<bf16,f32> (scatter-accumulate)",
            "bound": "hbm",
            "achieved": round(accum_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(accum_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic.get("accum", (None, None))[0],
            "traffic_source": traffic.get("accum", (None, None))[1],
            "algorithmic_bytes": 10 * N,
            "avg_launch_ms": round(a_ms, 5),
            "median_launch_ms": round(statistics.median(durations["accum"]), 5),
            "min_launch_ms": round(min(durations["accum"]), 5),
            "max_launch_ms": round(max(durations["accum"]), 5),
            "launches_timed": len(durations["accum"]),
            "launch_ms_in_order": [round(x, 4) for x in durations["accum"][:2 * MICROBATCHES]],
            "practical_ceiling": ceiling,
        },
        "roofline_gather": {
            "kernel": "gather_kernel",
            "bound": "hbm",
            "achieved": round(gather_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(gather_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic.get("gather", (None, None))[0],
            "traffic_source": traffic.get("gather", (None, None))[1],
            "algorithmic_bytes": 4 * N,
            "avg_launch_ms": round(g_ms, 5),
            "median_launch_ms": round(statistics.median(durations["gather"]), 5),
            "min_launch_ms": round(min(durations["gather"]), 5),
            "launches_timed": len(durations["gather"]),
            "max_launch_ms": round(max(durations["gather"]), 5),
        },
        "clear": {"avg_launch_ms": round(c_ms, 5) if c_ms else None,
                  "GB/s": round(4 * N / (c_ms * 1e-3) / 1e9, 1) if c_ms else None},
        "store": {"avg_launch_ms": round(s_ms, 5) if s_ms else None,
                  "GB/s": round(6 * N / (s_ms * 1e-3) / 1e9, 1) if s_ms else None,
                  "traffic": traffic.get("store", (None, None))[0] if s_ms else None},
        "minibatch_ms": round(elapsed / args.steps * MICROBATCHES * 1e3, 4),
        "host_us_per_call": host_overhead,
        "launch_floor_us": launch_floor,
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
