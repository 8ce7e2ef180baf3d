"""FSDP glue on the GPU: the flat-parameter call sites and hooks (fsdp1) and the parameter-group
layout with fused and two-step data flow (fsdp2), against the CPU oracle."""

import math
import types

import pytest
import torch

from helpers import assert_bit_equal, put_shards
from oracle import odc_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["eager", "lazy"], autouse=True)
def clear_mode(request, monkeypatch):
    """Every test here runs with the reference's eager clears (the default) and with lazy clears
    (ODC_LAZY_CLEAR=1, read when the FSDP patches build their ReductionService)."""
    monkeypatch.setenv("ODC_LAZY_CLEAR", "1" if request.param == "lazy" else "0")
    return request.param


def test_fsdp1_hooks_and_call_sites(make_world):
    """One minibatch the way examples/llm_training/torch_fsdp.py:462-481 drives it:
    pre_minibatch_start, per microbatch gather + reduce_grad for two flat params, then
    pre_optimizer_step publishes flat_param.grad = acc / factor in the parameter dtype."""
    import odc_amd
    from odc_amd.fsdp import fsdp1

    W, M = 8, 3
    group = make_world(W, 16 << 20)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    g = torch.Generator().manual_seed(1)
    numels = [100_003, 4096 * 8 + 5]
    fulls = [(torch.randn(n, generator=g) * 0.02).bfloat16() for n in numels]
    flat_params, handles = [], []
    for full in fulls:
        holder = torch.nn.Parameter(full.clone().cuda(), requires_grad=False)
        for r in range(W):
            sharded, pad = fsdp1.get_shard(holder, r, W)
            assert_bit_equal(sharded, oracle.fsdp1_get_shard(full, r, W), f"shard {r}")
        local = odc_amd.SymmBufferRegistry.get_instance().get_symm_buffer(id(holder))
        holder.data = local  # FSDP points flat_param.data at the local shard
        flat = types.SimpleNamespace(data=local, holder=holder)
        flat_params.append(flat)
        handles.append(types.SimpleNamespace(flat_param=holder))
    module = types.SimpleNamespace(process_group=group, _gradient_postdivide_factor=float(W), _all_handles=handles)

    fsdp1.pre_minibatch_start(module)
    want = [[torch.zeros(math.ceil(n / W)) for _ in range(W)] for n in numels]
    for _ in range(M):
        for i, (flat, full) in enumerate(zip(flat_params, fulls)):
            S = math.ceil(numels[i] / W)
            out = torch.empty(W * S, dtype=torch.bfloat16, device="cuda")
            fsdp1.all_gather_flat_param(out, flat.data, group)
            assert_bit_equal(out[: numels[i]], full, "gathered flat param")
            grad = (torch.randn(numels[i], generator=g) * 1e-3).bfloat16()
            saved = fsdp1.reduce_grad(flat.holder, grad.cuda(), group)
            assert saved.data_ptr() == fsdp1.get_reduction_service().get_accumulation(id(flat.holder)).data_ptr()
            oracle.scatter_accumulate(want[i], oracle.fsdp1_pad_grad(grad, W))
    fsdp1.pre_optimizer_step(module)
    for i, handle in enumerate(handles):
        expect = oracle.fsdp1_publish(want[i][0].clone(), float(W), torch.bfloat16)
        assert handle.flat_param.grad.dtype == torch.bfloat16
        assert_bit_equal(handle.flat_param.grad, expect, f"published grad {i}")
    # the next minibatch starts from zero again
    fsdp1.pre_minibatch_start(module)
    fsdp1.get_reduction_service().sync(group)
    for h in handles:
        acc = fsdp1.get_reduction_service().get_accumulation(id(h.flat_param))
        assert not acc.cpu().any()
    # stop() tears everything down (fsdp1.py:345-348)
    from odc_amd.primitives import utils

    for h in handles:
        h.flat_param.data = torch.empty(0)  # drop the views into the arena first
        h.flat_param.grad = None
    fsdp1.stop()
    assert not utils.is_initialized() and not odc_amd.SymmBufferRegistry.get_instance().has_key(id(handles[0].flat_param))


@pytest.mark.parametrize("W", [4, 8, 12])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_fsdp2_group_layout(make_world, W, fused, dtype):
    """A parameter group with uneven dim 0 (padding rows, empty tail shards): unshard and reduce,
    fused and two-step, equal the oracle built from torch._chunk_cat / split_with_sizes_copy."""
    from odc_amd import virtual_rank
    from odc_amd.fsdp import fsdp2

    group = make_world(W, 32 << 20)
    fsdp2.patch_fsdp2()
    fsdp2.reduction_service.accumulation_dtype = None
    shapes = [(37, 24), (5,), (64, 16), (3, 7, 2), (1024, 96), (W + 1, 33)]
    g = torch.Generator().manual_seed(W)
    params = [(torch.randn(*s, generator=g) * 0.02).to(dtype) for s in shapes]
    pgp = fsdp2.ParamGroup(shapes, dtype, group, reduce_dtype=torch.float32, name="blk")
    pgp.load_full_params([p.cuda() for p in params])

    packed = oracle.fsdp2_pack_shards(params, W)
    from odc_amd import SymmBufferRegistry

    for r, buf in enumerate(SymmBufferRegistry.get_instance().peer_tensors[pgp.key]):
        assert_bit_equal(buf, packed[r], f"packed shard of rank {r}")
    unsharded = pgp.unshard(fused=fused)
    want = oracle.fsdp2_copy_out(oracle.gather(packed), shapes, W)
    for p, (u, w, full) in enumerate(zip(unsharded, want, params)):
        assert_bit_equal(u, w, f"unsharded param {p}")
        assert_bit_equal(u, full, f"unsharded param {p} vs original")

    module = types.SimpleNamespace(_odc_param_groups=[pgp])
    fsdp2.pre_minibatch_start(module)
    accs = [torch.zeros(pgp.total_shard_numel) for _ in range(W)]
    for _ in range(3):
        grads = [(torch.randn(*s, generator=g) * 1e-3).to(dtype) for s in shapes]
        pgp.reduce([x.cuda() for x in grads], fused=fused)
        oracle.scatter_accumulate(accs, oracle.fsdp2_copy_in(grads, W, torch.float32))
    for r in range(W):
        with virtual_rank(r):
            if r == 0:
                fsdp2.pre_optimizer_step(module)
                got = pgp.sharded_grads
            else:
                pgp._reduced = True
                got = pgp.update_gradients()
            wantv = oracle.fsdp2_grad_views(oracle.fsdp2_average(accs[r].clone(), W).to(dtype), shapes, W, r)
            for p, (a, b) in enumerate(zip(got, wantv)):
                assert tuple(a.shape) == tuple(b.shape), f"rank {r} param {p}"
                assert_bit_equal(a.contiguous(), b.contiguous(), f"rank {r} sharded grad {p}")
    assert set(fsdp2.get_symm_buffer_memory_breakdown()) >= {"fsdp_params", "accumulation"}
    from odc_amd.primitives import utils

    del got, unsharded, pgp
    fsdp2.stop()  # fsdp2.py:1141-1144
    assert not utils.is_initialized()


def test_fsdp2_group_gathers_from_shards_kept_in_the_compute_dtype(make_world):
    """fp32 shards, bf16 compute, ``compute_dtype_shards=True``: the group keeps a bf16 copy of
    every rank's shards, converts it once per change of the shards and gathers from it. The
    unsharded parameters are bit-equal to converting on the way; an in-place update through torch
    is seen without any hook; one that bypasses torch's version counters is seen after the hook."""
    from odc_amd import SymmBufferRegistry
    from odc_amd.fsdp import fsdp2

    W = 4
    group = make_world(W, 32 << 20)
    fsdp2.patch_fsdp2()
    shapes = [(37, 24), (5,), (1024, 96), (W + 1, 33)]
    g = torch.Generator().manual_seed(5)
    params = [torch.randn(*s, generator=g) * 0.02 for s in shapes]
    kept = fsdp2.ParamGroup(shapes, torch.float32, group, param_dtype=torch.bfloat16, compute_dtype_shards=True)
    plain = fsdp2.ParamGroup(shapes, torch.float32, group, param_dtype=torch.bfloat16)
    for pgp in (kept, plain):
        pgp.load_full_params([p.cuda() for p in params])
    service = fsdp2.get_gather_service()
    conversions = []
    convert = service.convert_symm_buffer
    service.convert_symm_buffer = lambda *a, **k: (conversions.append(a), convert(*a, **k))[1]

    def check(what, n_conversions):
        for _ in range(3):  # three unshards, one conversion
            got = kept.unshard()
        want = plain.unshard()
        for p, (a, b) in enumerate(zip(got, want)):
            assert a.dtype == torch.bfloat16
            assert_bit_equal(a, b, f"{what}: unsharded param {p}")
        assert len(conversions) == n_conversions, what
        return got

    got = check("fresh", 1)
    for p, full in enumerate(params):
        assert_bit_equal(got[p], full.to(torch.bfloat16), f"unsharded param {p} vs original")
    registry = SymmBufferRegistry.get_instance()
    copy_key = kept.key + "_as_bfloat16"
    assert registry.has_key(copy_key) and registry.offsets[copy_key][2] == torch.bfloat16
    assert not registry.has_key(plain.key + "_as_bfloat16")

    # an optimizer step through torch (in place, on every rank's shards): seen by the version counters
    for pgp in (kept, plain):
        for r in range(W):
            for shard in pgp.sharded_params(r):
                shard.mul_(1.5).add_(0.001)
    check("after an in-place update", 2)
    check("unchanged shards", 2)

    # a write that torch's version counters do not see: the minibatch hook makes the copy anew
    for pgp in (kept, plain):
        for buf in registry.peer_tensors[pgp.key]:
            buf.data.mul_(-0.5)
    fsdp2.pre_minibatch_start(types.SimpleNamespace(_odc_param_groups=[kept, plain]))
    check("after the hook", 3)
    # ... and so does the documented invalidation call on its own
    import odc_amd.fsdp

    for pgp in (kept, plain):
        for r in range(W):
            for shard in pgp.sharded_params(r):
                shard.data.add_(0.25)  # .data: a detached alias with a version counter of its own
    odc_amd.fsdp.shards_may_have_changed()
    check("after shards_may_have_changed()", 4)
    # loading full parameters invalidates by itself
    for pgp in (kept, plain):
        pgp.load_full_params([p.cuda() * 2 for p in params])
    check("after load_full_params", 5)
    del got
    fsdp2.stop()


def test_group_paths_example_runs():
    """examples/fsdp2_group_paths.py (reference data flow against the fused one, timed) runs to
    the end; equality of the two flows is what test_fsdp2_group_layout checks."""
    import subprocess
    import sys
    from pathlib import Path

    script = Path(__file__).resolve().parent.parent / "examples" / "fsdp2_group_paths.py"
    proc = subprocess.run([sys.executable, str(script), "--iters", "3"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "publish" in proc.stdout and "unshard" in proc.stdout


def test_odc_all_gather_comm_object(make_world):
    """``ODCAllGather`` (fsdp2.py:76-90): torch's pluggable all-gather protocol over the gather
    primitive, synchronous and with the work handle of ``async_op=True``."""
    from odc_amd import SymmBufferRegistry
    from odc_amd.fsdp import fsdp2
    from torch.distributed.fsdp._fully_shard._fsdp_api import AllGather

    W, S = 8, 10_007
    group = make_world(W, 4 << 20)
    fsdp2.patch_fsdp2()
    try:
        comm = fsdp2.get_odc_gather_comm()
        assert isinstance(comm, AllGather) and comm is fsdp2.get_odc_gather_comm()
        g = torch.Generator().manual_seed(2)
        shards = [torch.randn(S, generator=g) for _ in range(W)]
        src = put_shards(SymmBufferRegistry.get_instance(), "ag", shards)
        out = comm.allocate((W * S,), dtype=torch.float32, device=torch.device("cuda"))
        assert comm(out, src, group) is None
        assert_bit_equal(out, oracle.gather(shards), "synchronous form")
        out.zero_()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            work = comm(out, src, group, async_op=True)
        assert work.wait()
        assert_bit_equal(out, oracle.gather(shards), "async form after wait()")
    finally:
        fsdp2.unpatch_fsdp2()


def test_record_function_ranges_become_marker_ranges_under_trace(monkeypatch):
    """``ODC_TRACE=1``: ``patch_fsdp2`` installs a ``record_function`` that also opens a marker
    range, in the three places the reference patches (fsdp2.py:1131-1133); the ranges still nest
    and close, and ``unpatch_fsdp2`` puts torch's class back. Without the switch nothing changes."""
    import torch.autograd.profiler
    import torch.profiler
    from torch.distributed.fsdp._fully_shard import _fsdp_param_group

    from odc_amd.fsdp import fsdp2

    original = torch.autograd.profiler.record_function
    homes = (_fsdp_param_group, torch.profiler, torch.autograd.profiler)
    fsdp2.patch_fsdp2()
    assert all(h.record_function is original for h in homes)
    fsdp2.unpatch_fsdp2()
    monkeypatch.setenv("ODC_TRACE", "1")
    fsdp2.patch_fsdp2()
    try:
        patched = _fsdp_param_group.record_function
        assert patched is not original and issubclass(patched, original)
        assert all(h.record_function is patched for h in homes)
        pushed = []
        monkeypatch.setattr(torch.cuda.nvtx, "range_push", lambda name: pushed.append(("push", name)))
        monkeypatch.setattr(torch.cuda.nvtx, "range_pop", lambda: pushed.append(("pop",)))
        with torch.profiler.record_function("FSDP::outer"):
            with _fsdp_param_group.record_function("FSDP::inner"):
                torch.ones(4, device="cuda").sum()
        assert pushed == [("push", "FSDP::outer"), ("push", "FSDP::inner"), ("pop",), ("pop",)]
    finally:
        fsdp2.unpatch_fsdp2()
    assert all(h.record_function is original for h in homes)
