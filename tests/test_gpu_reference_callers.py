"""Caller conformance: every place where the reference's own code calls into the primitives
(its FSDP patches and its two primitive examples) is replayed here with the reference's exact
attribute names, positional argument order and return conventions, against this package, on the
GPU, and checked against the CPU oracle or a closed form.

Each test names the reference lines it replays; CALL_SITES maps every call site to its test and
is checked to be complete.
"""

import pytest
import torch

import odc_amd as odc
from odc_amd.fsdp import fsdp1, fsdp2
from odc_amd.primitives import GatherService, ReductionService, SymmBufferRegistry
from oracle import odc_oracle as oracle

from helpers import assert_bit_equal

pytestmark = pytest.mark.gpu

W = 4

# reference call site -> test in this file
CALL_SITES = {
    "odc/fsdp/fsdp1.py:73-77": "test_fsdp1_reduce_grad_call_shape",
    "odc/fsdp/fsdp1.py:209-215": "test_fsdp1_all_gather_call_shape",
    "odc/fsdp/fsdp1.py:244-246": "test_fsdp1_get_shard_publishes_into_the_registry",
    "odc/fsdp/fsdp1.py:321": "test_fsdp1_pre_optimizer_step_calls",
    "odc/fsdp/fsdp1.py:324": "test_fsdp1_pre_optimizer_step_calls",
    "odc/fsdp/fsdp1.py:332-334": "test_fsdp1_pre_optimizer_step_calls",
    "odc/fsdp/fsdp1.py:339": "test_fsdp1_pre_minibatch_start_call",
    "odc/fsdp/fsdp1.py:346-348": "test_stop_sequence",
    "odc/fsdp/fsdp2.py:84-85": "test_fsdp2_odc_all_gather_call_shape",
    "odc/fsdp/fsdp2.py:157-159": "test_fsdp2_group_buffer_creation_and_views",
    "odc/fsdp/fsdp2.py:171-173": "test_fsdp2_group_buffer_creation_and_views",
    "odc/fsdp/fsdp2.py:261-264": "test_fsdp2_lookup_of_the_group_buffer",
    "odc/fsdp/fsdp2.py:709-710": "test_fsdp2_reduce_call_shape",
    "odc/fsdp/fsdp2.py:839-841": "test_fsdp2_update_gradients_divides_the_live_accumulation",
    "odc/fsdp/fsdp2.py:1039": "test_fsdp2_update_gradients_divides_the_live_accumulation",
    "odc/fsdp/fsdp2.py:1137-1138": "test_fsdp2_service_construction",
    "odc/fsdp/fsdp2.py:1142-1144": "test_stop_sequence",
    "odc/fsdp/fsdp2.py:1158": "test_fsdp2_memory_breakdown_reads_local_tensor",
    "examples/all_gather.py:84": "test_example_all_gather",
    "examples/all_gather.py:86": "test_example_all_gather",
    "examples/all_gather.py:112": "test_example_all_gather",
    "examples/reduce_scatter.py:52": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:108": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:116": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:122": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:164": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:169": "test_example_reduce_scatter",
    "examples/reduce_scatter.py:190": "test_example_reduce_scatter",
}


def test_every_call_site_has_a_test():
    for site, name in CALL_SITES.items():
        assert callable(globals().get(name)), f"{site} -> {name} is missing"


def _div_if_needed(tensor, div_factor):  # torch/distributed/fsdp/_runtime_utils.py, as the reference imports it
    if div_factor > 1:
        tensor.div_(div_factor)


class _Handle:
    def __init__(self, flat_param):
        self.flat_param = flat_param


class _FsdpState:
    """The attributes the reference reads from torch's _FSDPState (fsdp1.py:317-335)."""

    def __init__(self, pg, handles, postdivide=1.0):
        self.process_group = pg
        self._all_handles = handles
        self._gradient_postdivide_factor = postdivide


# ---------------------------------------------------------------------------------------------
# odc/fsdp/fsdp1.py
# ---------------------------------------------------------------------------------------------
def test_fsdp1_reduce_grad_call_shape(make_world):
    """fsdp1.py:73-77: rs_func = get_reduction_service().scatter_accumulate;
    rs_func(id(flat_param), padded_unsharded_grad, pg); get_accumulation(id(flat_param))."""
    pg = make_world(W, 8 << 20)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    flat_param = torch.nn.Parameter(torch.zeros(W * 1000, device="cuda"))
    g = torch.Generator().manual_seed(1)
    want = [torch.zeros(1000) for _ in range(W)]
    for _ in range(3):
        padded_unsharded_grad = (torch.randn(W * 1000, generator=g) * 1e-3).bfloat16()
        rs_func = fsdp1.get_reduction_service().scatter_accumulate
        assert rs_func(id(flat_param), padded_unsharded_grad.cuda(), pg) is None
        saved = fsdp1.get_reduction_service().get_accumulation(id(flat_param))
        oracle.scatter_accumulate(want, padded_unsharded_grad)
    assert saved.dtype == torch.float32 and saved.shape == (1000,)
    fsdp1.get_reduction_service().sync(pg)
    assert_bit_equal(saved, want[odc.get_rank()], "rank 0 accumulation")
    # the returned tensor IS the buffer: a later accumulate shows through it
    more = torch.ones(W * 1000, dtype=torch.bfloat16)
    fsdp1.get_reduction_service().scatter_accumulate(id(flat_param), more.cuda(), pg)
    oracle.scatter_accumulate(want, more)
    assert_bit_equal(saved, want[0], "live view")


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_fsdp1_all_gather_call_shape(make_world, out_dtype):
    """fsdp1.py:209-215: ag_func = gather_service.gather_into_tensor;
    ag_func(padded_unsharded_flat_param_orig_dtype, sharded_flat_param, pg) with fp32 shards."""
    pg = make_world(W, 8 << 20)
    fsdp1.patch_fsdp1()
    registry = SymmBufferRegistry.get_instance()
    g = torch.Generator().manual_seed(2)
    shards = [torch.randn(777, generator=g) for _ in range(W)]
    for r in range(W):
        with odc.virtual_rank(r):
            sharded_flat_param = registry.update_symm_buffer("flat", shards[r].cuda())
    sharded_flat_param = registry.get_symm_buffer("flat")
    padded_unsharded = torch.empty(W * 777, dtype=out_dtype, device="cuda")
    ag_func = fsdp1.get_gather_service().gather_into_tensor
    assert ag_func(padded_unsharded, sharded_flat_param, pg) is None
    assert_bit_equal(padded_unsharded, torch.cat(shards).to(out_dtype), "gathered flat parameter")


def test_fsdp1_get_shard_publishes_into_the_registry(make_world):
    """fsdp1.py:244-246: sharded_in_nvshmem = SymmBufferRegistry.get_instance()
    .update_symm_buffer(id(tensor), sharded) returns the symmetric tensor holding the shard."""
    make_world(W, 8 << 20)
    tensor = torch.arange(10, dtype=torch.float32, device="cuda")
    sharded = tensor[:3].clone()
    sharded_in_symm = odc.SymmBufferRegistry.get_instance().update_symm_buffer(id(tensor), sharded)
    assert SymmBufferRegistry.is_nvshmem_tensor(sharded_in_symm)
    assert sharded_in_symm.data_ptr() != sharded.data_ptr()
    assert_bit_equal(sharded_in_symm, sharded, "shard copy")
    # a second update before flush() keeps the first values (utils.py:103-116)
    again = odc.SymmBufferRegistry.get_instance().update_symm_buffer(id(tensor), sharded + 1)
    assert again.data_ptr() == sharded_in_symm.data_ptr()
    assert_bit_equal(again, sharded, "copy-once")
    assert len(odc.SymmBufferRegistry.get_instance().get_peer_tensors(sharded_in_symm)) == W


@pytest.mark.parametrize("lazy", [False, True])
def test_fsdp1_pre_optimizer_step_calls(make_world, lazy):
    """fsdp1.py:321,324,332-334, written as the reference writes them: sync(process_group); for
    acc in accumulations: _div_if_needed(acc, factor); flat_param.grad = get_accumulation(id).to(dtype)."""
    pg = make_world(W, 8 << 20)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    service = fsdp1.get_reduction_service()
    service.lazy_clear = lazy
    # between forward/backward a flat parameter is the local shard; its gradient is the full, padded one
    flat_params = [torch.nn.Parameter(torch.zeros(n, dtype=torch.bfloat16, device="cuda")) for n in (640, 96)]
    g = torch.Generator().manual_seed(3)
    want = {id(p): [torch.zeros(p.numel()) for _ in range(W)] for p in flat_params}
    for minibatch in range(2):
        service.clear_accumulations()
        for acc_list in want.values():
            for a in acc_list:
                a.zero_()
        touched = flat_params if minibatch == 0 else flat_params[:1]  # the second one stays cleared
        for _ in range(2):
            for p in touched:
                grad = (torch.randn(W * p.numel(), generator=g) * 1e-2).bfloat16()
                service.scatter_accumulate(id(p), grad.cuda(), pg)
                oracle.scatter_accumulate(want[id(p)], grad)
        fsdp_module = _FsdpState(pg, [_Handle(p) for p in flat_params], postdivide=4.0)  # a power of two: torch's device div_ and the CPU agree bit for bit
        # --- the reference's lines ---
        fsdp1.get_reduction_service().sync(fsdp_module.process_group)
        seen = 0
        for acc in fsdp1.get_reduction_service().accumulations:
            _div_if_needed(acc, fsdp_module._gradient_postdivide_factor)
            seen += 1
        for handle in fsdp_module._all_handles:
            handle.flat_param.grad = (
                fsdp1.get_reduction_service().get_accumulation(id(handle.flat_param)).to(handle.flat_param.dtype)
            )
        # -----------------------------
        assert seen == len(flat_params) == len(service.accumulations)
        for p in flat_params:
            expect = want[id(p)][0].clone().div_(4.0)
            assert_bit_equal(service.get_accumulation(id(p)), expect, f"minibatch {minibatch}: divided accumulation")
            assert_bit_equal(p.grad, expect.to(torch.bfloat16), f"minibatch {minibatch}: published grad")
            p.grad = None


@pytest.mark.parametrize("lazy", [False, True])
def test_fsdp1_pre_minibatch_start_call(make_world, lazy):
    """fsdp1.py:339: get_reduction_service().clear_accumulations() — afterwards every entry of
    `accumulations` reads as +0."""
    pg = make_world(W, 8 << 20)
    fsdp1.patch_fsdp1(reduce_dtype=torch.float32)
    service = fsdp1.get_reduction_service()
    service.lazy_clear = lazy
    service.scatter_accumulate("a", torch.ones(W * 300, dtype=torch.bfloat16, device="cuda"), pg)
    service.scatter_accumulate("b", torch.ones(W * 64, dtype=torch.bfloat16, device="cuda"), pg)
    assert fsdp1.get_reduction_service().clear_accumulations() is None
    for acc in service.accumulations:
        assert_bit_equal(acc, torch.zeros(acc.shape), "cleared accumulation")


def test_stop_sequence(make_world):
    """fsdp1.py:346-348 and fsdp2.py:1142-1144: get_reduction_service().stop();
    SymmBufferRegistry.get_instance().finalize(); finalize_distributed()."""
    pg = make_world(W, 8 << 20)
    fsdp2.patch_fsdp2()
    fsdp2.get_reduction_service().scatter_accumulate(0, torch.ones(W * 8, device="cuda"), pg)
    assert fsdp2.get_reduction_service().stop() is None
    SymmBufferRegistry.get_instance().finalize()
    assert SymmBufferRegistry.get_instance().memory_allocated() == 0
    odc.finalize_distributed()
    with pytest.raises(RuntimeError):
        odc.get_rank()  # the world is gone


# ---------------------------------------------------------------------------------------------
# odc/fsdp/fsdp2.py
# ---------------------------------------------------------------------------------------------
def test_fsdp2_service_construction(make_world):
    """fsdp2.py:1137-1138: ReductionService() and GatherService() without arguments; the
    accumulation then takes the gradient's dtype (scatter_accumulate.py:596-598)."""
    pg = make_world(W, 8 << 20)
    reduction_service, gather_service = ReductionService(), GatherService()
    assert reduction_service.accumulation_dtype is None and len(reduction_service.accumulations) == 0
    assert reduction_service.accumulation_indices == {} and reduction_service.dispatched_tasks == 0
    assert hasattr(gather_service, "buffer_splitter") and hasattr(reduction_service, "buffer_splitter")
    reduction_service.scatter_accumulate("k", torch.ones(W * 16, dtype=torch.bfloat16, device="cuda"), pg)
    assert reduction_service.get_accumulation("k").dtype == torch.bfloat16
    assert reduction_service.accumulation_indices == {"k": 0}


def test_fsdp2_odc_all_gather_call_shape(make_world):
    """fsdp2.py:84-85: gather = get_gather_service(); gather.gather_into_tensor(output_tensor,
    input_tensor, group), through ODCAllGather.__call__(output, input, group, async_op)."""
    pg = make_world(W, 8 << 20)
    fsdp2.patch_fsdp2()
    registry = SymmBufferRegistry.get_instance()
    g = torch.Generator().manual_seed(4)
    shards = [(torch.randn(1000, generator=g) * 0.02).bfloat16() for _ in range(W)]
    for r in range(W):
        with odc.virtual_rank(r):
            registry.update_symm_buffer("grp", shards[r].cuda())
    input_tensor = registry.get_symm_buffer("grp")
    comm = fsdp2.get_odc_gather_comm()
    output_tensor = comm.allocate((input_tensor.numel() * W,), dtype=input_tensor.dtype, device=input_tensor.device)
    assert comm(output_tensor, input_tensor, pg) is None
    assert_bit_equal(output_tensor, torch.cat(shards), "ODCAllGather")
    output_tensor.zero_()
    work = comm(output_tensor, input_tensor, pg, async_op=True)
    assert work is not None
    work.wait()
    assert_bit_equal(output_tensor, torch.cat(shards), "ODCAllGather async")


def test_fsdp2_group_buffer_creation_and_views(make_world):
    """fsdp2.py:157-159,171-173,186-196: get_or_create_symm_buffer(key, (total_size,), dtype),
    then symm_buffer[offset : offset + n].copy_(shard), .view(padded size), .narrow(dim, 0, length)."""
    make_world(W, 8 << 20)
    registry = SymmBufferRegistry.get_instance()
    key = "fsdp_params_gather_1_2"
    sizes = [(3, 5), (2, 7)]
    total_size = sum(a * b for a, b in sizes)
    symm_buffer = registry.get_or_create_symm_buffer(key, (total_size,), torch.float32)
    assert symm_buffer.shape == (total_size,) and symm_buffer.dtype == torch.float32 and symm_buffer.is_cuda
    assert registry.get_or_create_symm_buffer(key, (total_size,), torch.float32).data_ptr() == symm_buffer.data_ptr()
    offset, params = 0, []
    for a, b in sizes:
        data = torch.randn(a * b, device="cuda")
        symm_buffer[offset : offset + a * b].copy_(data)
        padded_sharded_param = symm_buffer[offset : offset + a * b].view((a, b))
        sharded_param = padded_sharded_param.narrow(dim=0, start=0, length=a - 1)
        params.append((data, padded_sharded_param, sharded_param))
        offset += a * b
    for (data, padded, narrow), (a, b) in zip(params, sizes):
        assert_bit_equal(padded.reshape(-1), data, "view of the group buffer")
        assert narrow.shape == (a - 1, b) and narrow.data_ptr() == padded.data_ptr()
    # the keyed buffer still resolves to the same W peers
    assert len(registry.get_peer_tensors(symm_buffer)) == W
    # an hpz-style second buffer under its own key (fsdp2.py:171-173) is independent
    hpz = registry.get_or_create_symm_buffer("hpz_" + key, (2 * total_size,), torch.bfloat16)
    assert hpz.numel() == 2 * total_size and hpz.data_ptr() != symm_buffer.data_ptr()


def test_fsdp2_lookup_of_the_group_buffer(make_world):
    """fsdp2.py:261-264: assert registry.has_key(key); all_gather_input = registry.get_symm_buffer(key)."""
    make_world(W, 8 << 20)
    registry = SymmBufferRegistry.get_instance()
    key = "fsdp_params_gather_7"
    assert not SymmBufferRegistry.get_instance().has_key(key)
    with pytest.raises(ValueError):
        registry.get_symm_buffer(key)  # utils.py:153-156
    made = registry.get_or_create_symm_buffer(key, (128,), torch.bfloat16)
    assert SymmBufferRegistry.get_instance().has_key(key)
    all_gather_input = SymmBufferRegistry.get_instance().get_symm_buffer(key)
    assert all_gather_input.data_ptr() == made.data_ptr() and all_gather_input.numel() == 128
    with pytest.raises(AssertionError):
        registry.allocate_symm_buffer(key, (128,), torch.bfloat16)  # utils.py:127


def test_fsdp2_reduce_call_shape(make_world):
    """fsdp2.py:709-710: key = id(fsdp_param_group); scatter = get_reduction_service();
    scatter.scatter_accumulate(key, reduce_scatter_input, reduce_scatter_group) with the fp32
    reduce-scatter input that chunk_cat produced."""
    pg = make_world(W, 8 << 20)
    fsdp2.patch_fsdp2()
    fsdp_param_group = object()
    key = id(fsdp_param_group)
    g = torch.Generator().manual_seed(5)
    grads = [torch.randn(6, 5, generator=g), torch.randn(3, 4, generator=g)]  # dim 0 not divisible by W
    shard_numel = sum(-(-t.shape[0] // W) * t.shape[1] for t in grads)
    want = [torch.zeros(shard_numel) for _ in range(W)]
    for _ in range(2):
        reduce_scatter_input = torch.empty(W * shard_numel)
        torch._chunk_cat(grads, dim=0, num_chunks=W, out=reduce_scatter_input.view(W, -1))
        scatter = fsdp2.get_reduction_service()
        assert scatter.scatter_accumulate(key, reduce_scatter_input.cuda(), pg) is None
        oracle.scatter_accumulate(want, reduce_scatter_input)
    scatter.sync(pg)
    for r, acc in enumerate(scatter.get_peer_accumulations(key)):
        assert_bit_equal(acc, want[r], f"rank {r}")


@pytest.mark.parametrize("lazy", [False, True])
def test_fsdp2_update_gradients_divides_the_live_accumulation(make_world, lazy):
    """fsdp2.py:1039 and 839-841,846-847: scatter.sync(group); reduce_output =
    scatter.get_accumulation(key); reduce_output /= world_size — in place, on the buffer itself;
    then strided views of it become the gradients (fsdp2.py:902-907)."""
    pg = make_world(W, 8 << 20)
    fsdp2.patch_fsdp2()
    scatter = fsdp2.get_reduction_service()
    scatter.lazy_clear = lazy
    key = id(pg)
    grad = torch.arange(W * 24, dtype=torch.float32)
    scatter.clear_accumulations()
    scatter.scatter_accumulate(key, grad.cuda(), pg)
    scatter.scatter_accumulate(key, grad.cuda(), pg)
    scatter.sync(pg)
    reduce_output = scatter.get_accumulation(key)
    world_size = pg.size()
    reduce_output /= world_size
    want = (grad.view(W, -1)[0] * 2) / W
    assert_bit_equal(scatter.get_accumulation(key), want, "in-place division reaches the buffer")
    assert_bit_equal(scatter.accumulations[scatter.accumulation_indices[key]], want, "accumulations[index]")
    sharded_grad = torch.as_strided(reduce_output, size=(4, 3), stride=(3, 1), storage_offset=12)
    assert_bit_equal(sharded_grad, want[12:24].view(4, 3), "strided gradient view")


def test_fsdp2_memory_breakdown_reads_local_tensor(make_world):
    """fsdp2.py:1158: for key, tensor in registry.local_tensor.items(): tensor.nbytes by prefix."""
    pg = make_world(W, 64 << 20)
    fsdp2.patch_fsdp2()
    registry = SymmBufferRegistry.get_instance()
    registry.get_or_create_symm_buffer("fsdp_params_gather_1", (1 << 20,), torch.float32)
    fsdp2.get_reduction_service().scatter_accumulate(9, torch.zeros(W << 19, device="cuda"), pg)
    sizes = {key: tensor.nbytes for key, tensor in registry.local_tensor.items()}
    assert sizes == {"fsdp_params_gather_1": 4 << 20, "rs_accumulation_9": 2 << 20}
    breakdown = fsdp2.get_symm_buffer_memory_breakdown()
    assert breakdown["fsdp_params"] == round((4 << 20) / 2**30, 2) and breakdown["accumulation"] == round((2 << 20) / 2**30, 2)
    assert registry.memory_allocated() == (4 << 20) + (2 << 20)


# ---------------------------------------------------------------------------------------------
# examples/all_gather.py, examples/reduce_scatter.py
# ---------------------------------------------------------------------------------------------
def test_example_all_gather(make_world):
    """all_gather.py:80-86,112,121-125: tensor i of rank r is filled with i + 2r and published
    with registry.update_symm_buffer(i, src); gather_service.gather_into_tensor(dst, src, group);
    block r of dst == 2r + i."""
    cnt, size, dtype = 5, 1 << 14, torch.int64
    group = make_world(W, cnt * size * 8 + (1 << 20))
    registry = SymmBufferRegistry.get_instance()
    src_tensors = [torch.empty(size, dtype=dtype, device="cuda") for _ in range(cnt)]
    for rank in range(W):  # each process of the reference does this once, as its own rank
        with odc.virtual_rank(rank):
            for i in range(cnt):
                filled = torch.empty(size, dtype=dtype, device="cuda").fill_(i + rank * 2)
                published = registry.update_symm_buffer(i, filled)
                if rank == 0:
                    src_tensors[i] = published
    gather_service = GatherService()
    group_ranks = list(range(W))
    for i in range(cnt):
        dst = torch.empty(size * W, dtype=dtype, device="cuda")
        all_gather_func = gather_service.gather_into_tensor
        all_gather_func(dst, src_tensors[i], group)
        for r in range(W):
            expected = group_ranks[r] * 2 + i
            assert torch.eq(dst[r * size : (r + 1) * size], expected).all()


@pytest.mark.parametrize("lazy", [False, True])
def test_example_reduce_scatter(make_world, lazy):
    """reduce_scatter.py:52,108,116,122,164-172,190: ReductionService(accumulation_dtype=...);
    clear_accumulations(); scatter_accumulate(dest_idx, src_tensor, pg) over `times` rounds;
    sync(group); assert_close(reference sums, reduction_service.accumulations[i], 5e-3, 5e-3);
    stop(). One client contributes on one GPU, so the reference sums are the client's own
    chunks, and the comparison is exact as well."""
    accum_dtype = grad_dtype = torch.float32
    cnt, times, size = 2, 5, 128 * 1024 + 1024
    group = make_world(W, cnt * (size // W) * 4 + (1 << 20))
    reduction_service = ReductionService(accumulation_dtype=accum_dtype, lazy_clear=lazy)
    g = torch.Generator().manual_seed(6)
    data = [torch.rand(size, dtype=grad_dtype, generator=g) for _ in range(cnt * times)]
    device_data = [d.cuda() for d in data]
    nccl_accumulations = [torch.zeros(size // W, dtype=accum_dtype) for _ in range(cnt)]

    def scatter_accumulation(src_tensor, dest_idx, pg):
        reduction_service.scatter_accumulate(dest_idx, src_tensor, pg)

    # the warm-up pass of the example, then the cleared, checked pass
    reduction_service.clear_accumulations()
    for i in range(cnt * times):
        scatter_accumulation(device_data[i], i % cnt, group)
    reduction_service.sync(group)
    reduction_service.clear_accumulations()
    for i in range(cnt * times):
        scatter_accumulation(device_data[i], i % cnt, group)
        nccl_accumulations[i % cnt].add_(data[i].view(W, -1)[0])  # reduce_scatter of one contributor + add_
    reduction_service.sync(group)
    for i in range(cnt):
        torch.testing.assert_close(
            nccl_accumulations[i].cuda(), reduction_service.accumulations[i], rtol=5e-3, atol=5e-3
        )
        assert_bit_equal(reduction_service.accumulations[i], nccl_accumulations[i], f"accumulations[{i}]")
    assert reduction_service.stop() is None


def test_the_reference_import_lines_work_unchanged(make_world):
    """The import statements of the reference's callers, verbatim (examples/all_gather.py:10-11,
    examples/reduce_scatter.py:9-10, examples/FSDP2/example.py:15-17, examples/llm_training's
    ``import odc`` / ``from odc.fsdp import fsdp1``), give the objects of this package, and the
    reference's known-answer gather (examples/all_gather.py:80-84,121-125: shard i of rank r holds
    i + 2r) runs through them."""
    import odc
    from odc import init_nvshmem
    from odc.fsdp import fsdp1 as ref_fsdp1
    from odc.fsdp import fsdp2 as ref_fsdp2
    from odc.primitives.gather import GatherService as RefGatherService
    from odc.primitives.scatter_accumulate import ReductionService as RefReductionService
    from odc.primitives.utils import SymmBufferRegistry as RefRegistry
    from odc.primitives.utils import finalize_distributed, get_local_world_size, init_nvshmem as init_from_utils

    import odc_amd
    import odc_amd.primitives.utils as amd_utils

    assert RefGatherService is GatherService and RefReductionService is ReductionService
    assert RefRegistry is SymmBufferRegistry and ref_fsdp1 is fsdp1 and ref_fsdp2 is fsdp2
    assert init_nvshmem is init_from_utils is odc_amd.init_nvshmem and odc.init_nvshmem is init_nvshmem
    assert finalize_distributed is amd_utils.finalize_distributed
    assert get_local_world_size is amd_utils.get_local_world_size
    assert odc.ReductionService is ReductionService and odc.primitives.utils is amd_utils

    group = make_world(W, 4 << 20)
    registry = RefRegistry.get_instance()
    gather = RefGatherService()
    n = 4096
    for r in range(W):
        with odc.virtual_rank(r):
            registry.update_symm_buffer(0, torch.full((n,), 0 + 2 * r, dtype=torch.int64, device="cuda"))
    out = torch.empty(W * n, dtype=torch.int64, device="cuda")
    gather.gather_into_tensor(out, registry.get_symm_buffer(0), group)
    for r in range(W):
        assert (out[r * n : (r + 1) * n] == 2 * r).all()
