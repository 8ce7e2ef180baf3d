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
items carry ``flat_param``), so they also serve stand-in modules. ``patch_fsdp1`` installs the call
sites into torch's ``FullyShardedDataParallel``; one process then plays one rank of a W-rank
process group (for instance torch's "fake" backend).
"""

from __future__ import annotations

import logging
import os

import torch
import torch.nn.functional as F

import odc_amd
from odc_amd.fsdp.shard_copies import compute_dtype_shards_of, shards_may_have_changed
from odc_amd.primitives.utils import group_size

logger = logging.getLogger(__name__)

reduction_service = None
gather_service = None
_compute_dtype_shards = False  # patch_fsdp1(compute_dtype_shards=...)


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


custom_get_shard = get_shard  # the reference's name for it (fsdp1.py:239)


def all_gather_flat_param(padded_unsharded_flat_param, sharded_flat_param, pg, param_dtype=None, watch=()):
    """Gather the padded flat parameter. The shards stay in their own dtype (a peer may not have
    produced a low-precision copy yet: that is why the reference gathers in the shard dtype into
    a temporary and casts afterwards, fsdp1.py:199-223); when the output dtype differs, the
    conversion happens inside the gather kernel, or, with ``patch_fsdp1(compute_dtype_shards=True)``,
    once per change of the shards into a copy that the gathers then read
    (``shard_copies.compute_dtype_shards_of``; ``watch``: the flat parameter, whose version
    counter the optimizer bumps)."""
    expected = sharded_flat_param.numel() * group_size(pg)
    assert (
        padded_unsharded_flat_param.numel() == expected
    ), f"Expects {expected} numel but got {padded_unsharded_flat_param.numel()}"
    if padded_unsharded_flat_param.dtype != sharded_flat_param.dtype:
        assert param_dtype in (None, padded_unsharded_flat_param.dtype)
        if _compute_dtype_shards and sharded_flat_param.numel():
            registry = odc_amd.SymmBufferRegistry.get_instance()
            key = registry.local_tensor_to_keys[sharded_flat_param.data_ptr()]
            sharded_flat_param = compute_dtype_shards_of(
                gather_service, key, sharded_flat_param.numel(), padded_unsharded_flat_param.dtype, watch=watch
            )
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


# ------------------------------------------------------------------------------------------------
# torch FullyShardedDataParallel integration (the monkey patches of fsdp1.py:302-314)
# ------------------------------------------------------------------------------------------------
_originals = {}


def _patched_get_shard(tensor, rank, world_size):
    """``FlatParamHandle._get_shard`` (fsdp1.py:239-247): the calling rank's padded chunk, living
    in its symmetric buffer. One process holds all W virtual ranks, so every rank's chunk is
    published here (in the reference each process publishes its own)."""
    from torch.distributed.fsdp._flat_param import FlatParameter

    assert isinstance(tensor, FlatParameter)
    registry = odc_amd.SymmBufferRegistry.get_instance()
    original = _originals["_get_shard"]
    local, local_pad = None, 0
    for r in range(world_size):
        sharded, numel_to_pad = original(tensor, r, world_size)
        with odc_amd.virtual_rank(r):
            in_symm = registry.update_symm_buffer(id(tensor), sharded)
        if r == rank:
            local, local_pad = in_symm, numel_to_pad
    return local, local_pad


def _patched_all_gather_flat_param(self, padded_unsharded_flat_param):
    """``FlatParamHandle._all_gather_flat_param`` (fsdp1.py:156-233)."""
    sharded_flat_param = self.flat_param.data
    pg = self._fake_process_group if self._use_fake_all_gather else self.process_group
    assert not sharded_flat_param.is_cpu and not self._offload_params, "ODC does not support offloading"
    return all_gather_flat_param(
        padded_unsharded_flat_param, sharded_flat_param, pg, param_dtype=self._fwd_bwd_param_dtype,
        watch=(self.flat_param,),
    )


def _patched_use_low_precision_shard(self):
    """No low-precision copy of the shard is made: peers read the shard in its own dtype and
    the gather converts (fsdp1.py:250-275)."""
    self._check_low_precision_shard()


def _patched_free_low_precision_sharded_param(self):
    self._check_low_precision_shard()  # nothing was allocated (fsdp1.py:278-299)


def _patched_reduce_grad(state, handle) -> None:
    """``_runtime_utils._reduce_grad`` (fsdp1.py:41-106)."""
    from torch.distributed.fsdp._flat_param import HandleShardingStrategy

    flat_param = handle.flat_param
    assert handle._sharding_strategy not in (
        HandleShardingStrategy.HYBRID_SHARD,
        HandleShardingStrategy._HYBRID_SHARD_ZERO2,
    ), "ODC does not support hybrid sharded strategy"
    assert state._comm_hook is None, "ODC does not support comm hook"
    assert not handle._offload_params, "ODC does not support offloading"
    assert not handle._use_orig_params, "ODC does not support using original parameters"
    unsharded_grad = flat_param.grad.data
    flat_param.grad = None  # permits several backwards per minibatch
    pg = handle._fake_process_group if handle._use_fake_reduce else state.process_group
    flat_param._saved_grad_shard = reduce_grad(
        flat_param, unsharded_grad, pg, predivide_factor=state._gradient_predivide_factor
    )


def _patched_prepare_gradient_for_optim(self):
    """``FlatParamHandle.prepare_gradient_for_optim`` (fsdp1.py:109-153): at the end of a backward
    the accumulation is NOT forwarded to ``.grad``; ``pre_optimizer_step`` publishes it."""
    flat_param = self.flat_param
    assert not hasattr(flat_param, "_cpu_grad"), "ODC does not support offloading"
    if hasattr(flat_param, "_saved_grad_shard"):
        self._check_sharded(flat_param)
        if flat_param._post_backward_called:
            flat_param.grad = None
        delattr(flat_param, "_saved_grad_shard")


def patch_fsdp1(reduce_dtype=None, compute_dtype_shards=None):
    """Create the two services and route torch FSDP1's all-gather and reduce-scatter through
    them (fsdp1.py:302-314). Call before wrapping modules: shards move into the symmetric arena
    when ``FullyShardedDataParallel`` shards its flat parameters.

    ``compute_dtype_shards`` (default: ``$ODC_FSDP1_COMPUTE_DTYPE_SHARDS == "1"``, off): under
    mixed precision, keep every flat parameter's shards a second time in the compute dtype and
    gather from that copy."""
    global reduction_service, gather_service, _compute_dtype_shards
    if compute_dtype_shards is None:
        compute_dtype_shards = os.environ.get("ODC_FSDP1_COMPUTE_DTYPE_SHARDS", "0") == "1"
    _compute_dtype_shards = bool(compute_dtype_shards)
    reduction_service = odc_amd.ReductionService(accumulation_dtype=reduce_dtype)
    gather_service = odc_amd.GatherService()
    from torch.distributed.fsdp import _runtime_utils
    from torch.distributed.fsdp._flat_param import FlatParamHandle

    if not _originals:
        _originals.update(
            _reduce_grad=_runtime_utils._reduce_grad,
            prepare_gradient_for_optim=FlatParamHandle.prepare_gradient_for_optim,
            _get_shard=FlatParamHandle._get_shard,
            _all_gather_flat_param=FlatParamHandle._all_gather_flat_param,
            _use_low_precision_shard=FlatParamHandle._use_low_precision_shard,
            _free_low_precision_sharded_param=FlatParamHandle._free_low_precision_sharded_param,
        )
    _runtime_utils._reduce_grad = _patched_reduce_grad
    FlatParamHandle.prepare_gradient_for_optim = _patched_prepare_gradient_for_optim
    FlatParamHandle._get_shard = staticmethod(_patched_get_shard)
    FlatParamHandle._all_gather_flat_param = _patched_all_gather_flat_param
    FlatParamHandle._use_low_precision_shard = _patched_use_low_precision_shard
    FlatParamHandle._free_low_precision_sharded_param = _patched_free_low_precision_sharded_param


def unpatch_fsdp1():
    """Put torch's own methods back (for running patched and unpatched in one process)."""
    if not _originals:
        return
    from torch.distributed.fsdp import _runtime_utils
    from torch.distributed.fsdp._flat_param import FlatParamHandle

    _runtime_utils._reduce_grad = _originals.pop("_reduce_grad")
    FlatParamHandle._get_shard = staticmethod(_originals.pop("_get_shard"))
    for name, fn in list(_originals.items()):
        setattr(FlatParamHandle, name, fn)
    _originals.clear()


def pre_optimizer_step(fsdp_module):
    """fsdp1.py:317-335: wait for every add, post-divide, publish the accumulations as
    ``flat_param.grad`` in the parameter dtype."""
    shards_may_have_changed()  # the optimizer is about to change them
    with torch.cuda.nvtx.range("scatter_accumulate_sync"):
        get_reduction_service().sync(getattr(fsdp_module, "process_group", None))
    if hasattr(fsdp_module, "_inter_node_pg"):
        raise NotImplementedError("hybrid sharding needs a second node; not part of this build")
    service = get_reduction_service()
    factor = getattr(fsdp_module, "_gradient_postdivide_factor", 1.0)
    divisor = factor if factor is not None and factor > 1 else 1.0  # `_div_if_needed`
    # a unit that never saw a gradient (frozen, or unused so far) has no accumulation yet
    handles = [h for h in fsdp_module._all_handles if id(h.flat_param) in service.accumulation_indices]
    by_dtype = {}  # one publish launch per (accumulation dtype, parameter dtype)
    for handle in handles:
        pair = (service.accumulation_dtype_of(id(handle.flat_param)), handle.flat_param.dtype)
        by_dtype.setdefault(pair, []).append(handle)
    published = set()
    for (_acc_dtype, dtype), group in by_dtype.items():
        keys = [id(h.flat_param) for h in group]
        for handle, grad in zip(group, service.publish(keys, out_dtype=dtype, divisor=divisor)):
            handle.flat_param.grad = grad
        published.update(keys)
    if divisor != 1.0:  # the reference divides every accumulation, handle or not (fsdp1.py:324-327)
        rest = {}
        for key in service.accumulation_keys:
            if key not in published:
                rest.setdefault(service.accumulation_dtype_of(key), []).append(key)
        for keys in rest.values():
            service.publish(keys, divisor=divisor)


def pre_minibatch_start(_fsdp_module):
    """fsdp1.py:338-342: zero the accumulations; the reference then barriers so that optimizer
    updates are visible to all ranks, which for ranks sharing one device is stream order."""
    shards_may_have_changed()
    get_reduction_service().clear_accumulations()
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        torch.distributed.barrier()


def stop():
    get_reduction_service().stop()
    odc_amd.SymmBufferRegistry.get_instance().finalize()
    odc_amd.finalize_distributed()
