"""FSDP1 (flat-parameter) glue: the three call sites and the two minibatch hooks.

Mirror of ``odc/fsdp/fsdp1.py``. The reference monkey-patches torch's ``FlatParamHandle`` and
``_runtime_utils._reduce_grad``; what those patches do on the hot path is three calls into the
primitives, provided here as plain functions with the same meaning:

    get_shard              <- custom_get_shard               (fsdp1.py:239-247)
    all_gather_flat_param  <- all_gather_flat_param           (fsdp1.py:156-233, the call at :209-215)
    reduce_grad            <- _reduce_grad                    (fsdp1.py:41-106, the calls at :25-38,65,73-77)

plus ``pre_minibatch_start`` / ``pre_optimizer_step`` / ``stop`` / ``patch_fsdp1`` with the
reference's signatures. The hooks take any object with the attributes the reference reads from
torch's ``_FSDPState`` (``process_group``, ``_gradient_postdivide_factor``, ``_all_handles`` whose
items carry ``flat_param``), so they also serve stand-in modules.
"""

from __future__ import annotations

import logging

import torch
import torch.nn.functional as F

import odc_amd
from odc_amd.primitives.utils import group_size

logger = logging.getLogger(__name__)

reduction_service = None
gather_service = None


def get_reduction_service():
    return reduction_service


def get_gather_service():
    return gather_service


def _div_if_needed(tensor: torch.Tensor, div_factor: float) -> None:
    # torch/distributed/fsdp/_runtime_utils.py `_div_if_needed`
    if div_factor is not None and div_factor > 1:
        tensor.div_(div_factor)


def get_shard(tensor: torch.Tensor, rank: int, world_size: int):
    """Rank ``rank``'s zero-padded chunk of the flat parameter, placed in (and returned as) its
    symmetric buffer keyed by ``id(tensor)``; second value is the number of padding elements.
    Chunking rule: torch/distributed/fsdp/_flat_param.py:1091-1142."""
    chunks = torch.flatten(tensor).chunk(world_size)
    chunk = chunks[rank] if rank < len(chunks) else chunks[0].new_empty(0)
    numel_to_pad = chunks[0].numel() - chunk.numel()
    sharded = F.pad(chunk, [0, numel_to_pad]) if numel_to_pad > 0 else chunk.clone()
    with odc_amd.virtual_rank(rank):
        sharded_in_symm = odc_amd.SymmBufferRegistry.get_instance().update_symm_buffer(
            id(tensor), sharded
        )
    return sharded_in_symm, numel_to_pad


def all_gather_flat_param(padded_unsharded_flat_param, sharded_flat_param, pg, param_dtype=None):
    """Gather the padded flat parameter. The shards stay in their own dtype (a peer may not have
    produced a low-precision copy yet: that is why the reference gathers in the shard dtype into
    a temporary and casts afterwards, fsdp1.py:199-223); when the output dtype differs, the
    conversion happens inside the gather kernel."""
    expected = sharded_flat_param.numel() * group_size(pg)
    assert (
        padded_unsharded_flat_param.numel() == expected
    ), f"Expects {expected} numel but got {padded_unsharded_flat_param.numel()}"
    if padded_unsharded_flat_param.dtype != sharded_flat_param.dtype:
        assert param_dtype in (None, padded_unsharded_flat_param.dtype)
    gather_service.gather_into_tensor(padded_unsharded_flat_param, sharded_flat_param, pg)
    return padded_unsharded_flat_param


def custom_get_reduce_scatter_tensors(world_size: int, unsharded_grad: torch.Tensor):
    """The padded gradient of fsdp1.py:25-38, materialised (kept for callers that want the
    tensor; ``reduce_grad`` itself never pads)."""
    chunks = list(unsharded_grad.chunk(world_size))
    numel_to_pad = world_size * chunks[0].numel() - unsharded_grad.numel()
    return F.pad(unsharded_grad, [0, numel_to_pad]) if numel_to_pad > 0 else unsharded_grad


def reduce_grad(flat_param, unsharded_grad: torch.Tensor, pg, predivide_factor: float = 1.0):
    """Scatter-accumulate one flat gradient under key ``id(flat_param)`` and return the calling
    rank's accumulation (what ``_reduce_grad`` stores as ``_saved_grad_shard``, fsdp1.py:73-77).
    The zero padding to W * ceil(numel / W) is applied inside the kernel."""
    W = group_size(pg)
    unsharded_grad = unsharded_grad.reshape(-1)
    _div_if_needed(unsharded_grad, predivide_factor)
    service = get_reduction_service()
    key = id(flat_param)
    shard = -(-unsharded_grad.numel() // W)
    if key not in service.accumulation_indices:
        accum_dtype = service.accumulation_dtype or unsharded_grad.dtype
        service.register(key, (shard,), unsharded_grad.dtype, accum_dtype, pg)
    service.scatter_accumulate_multi(
        [key], [unsharded_grad], pg, valid_numels=[unsharded_grad.numel()]
    )
    return service.get_accumulation(key)


def patch_fsdp1(reduce_dtype=None):
    """Create the two services (fsdp1.py:302-305). Rewiring torch's FlatParamHandle to call
    ``get_shard`` / ``all_gather_flat_param`` / ``reduce_grad`` needs a process group of W real
    ranks and is not done here."""
    global reduction_service, gather_service
    reduction_service = odc_amd.ReductionService(accumulation_dtype=reduce_dtype)
    gather_service = odc_amd.GatherService()


def pre_optimizer_step(fsdp_module):
    """fsdp1.py:317-335: wait for every add, post-divide, publish the accumulations as
    ``flat_param.grad`` in the parameter dtype."""
    with torch.cuda.nvtx.range("scatter_accumulate_sync"):
        get_reduction_service().sync(getattr(fsdp_module, "process_group", None))
    if hasattr(fsdp_module, "_inter_node_pg"):
        raise NotImplementedError("hybrid sharding needs a second node; not part of this build")
    service = get_reduction_service()
    factor = getattr(fsdp_module, "_gradient_postdivide_factor", 1.0)
    divisor = factor if factor is not None and factor > 1 else 1.0  # `_div_if_needed`
    handles = list(fsdp_module._all_handles)
    by_dtype = {}
    for handle in handles:
        by_dtype.setdefault(handle.flat_param.dtype, []).append(handle)
    published = set()
    for dtype, group in by_dtype.items():
        keys = [id(h.flat_param) for h in group]
        for handle, grad in zip(group, service.publish(keys, out_dtype=dtype, divisor=divisor)):
            handle.flat_param.grad = grad
        published.update(keys)
    rest = [k for k in service.accumulations if k not in published]
    if rest and divisor != 1.0:  # the reference divides every accumulation, handle or not
        service.publish(rest, divisor=divisor)


def pre_minibatch_start(_fsdp_module):
    """fsdp1.py:338-342: zero the accumulations; the reference then barriers so that optimizer
    updates are visible to all ranks, which for ranks sharing one device is stream order."""
    get_reduction_service().clear_accumulations()
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        torch.distributed.barrier()


def stop():
    get_reduction_service().stop()
    odc_amd.SymmBufferRegistry.get_instance().finalize()
    odc_amd.finalize_distributed()
