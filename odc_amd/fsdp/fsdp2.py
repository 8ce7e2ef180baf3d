"""FSDP2 (per-parameter, dim-0 sharded) glue: the parameter-group layout, its gather and
scatter-accumulate in one launch each, and the two minibatch hooks.

Mirror of the hot-path parts of ``odc/fsdp/fsdp2.py``:

    ParamGroup.load_full_params   <- replace_sharded_param_with_symm_buffer   (fsdp2.py:116-202)
    ParamGroup.unshard            <- foreach_all_gather + foreach_all_gather_copy_out
                                                                        (fsdp2.py:219-313, 317-424)
    ParamGroup.reduce             <- foreach_reduce                     (fsdp2.py:608-742)
    ParamGroup.update_gradients   <- update_gradients                   (fsdp2.py:795-957)
    pre_minibatch_start / pre_optimizer_step / patch_fsdp2 / stop / get_symm_buffer_memory_breakdown

Layout (fsdp2.py:146-196, torch/distributed/fsdp/_fully_shard/_fsdp_common.py:109-111): parameter
p of shape (d0, rest...) contributes ``n_p = ceil(d0 / W) * prod(rest)`` elements to every rank's
group buffer, rank r holding rows ``[r*ceil(d0/W), (r+1)*ceil(d0/W))`` zero padded; the group
buffer is the concatenation over p. The reference gathers it into ``[W, sum n_p]`` and then
copies out per parameter (and, the other way, ``chunk_cat``s gradients into ``[W, sum n_p]``
before the scatter-accumulate); ``fused=True`` (default) lets the kernels' work lists do both
directly, ``fused=False`` keeps the reference's two-step data flow.

HPZ (fsdp2.py:551-582, 745-791, 961-1099) and the HSDP all-reduce (fsdp2.py:849-885) need more
than one node and are not part of this build.
"""

from __future__ import annotations

import logging
import math
from typing import List, Optional, Sequence

import torch

from odc_amd.primitives.gather import GatherService
from odc_amd.primitives.scatter_accumulate import ReductionService
from odc_amd.primitives.utils import (
    SymmBufferRegistry,
    finalize_distributed,
    get_rank,
    group_size,
)

logger = logging.getLogger(__name__)

reduction_service = None
gather_service = None
_enable_hpz = None


def get_reduction_service():
    return reduction_service


def get_gather_service():
    return gather_service


def get_fsdp_params_key(ids: Sequence[int]) -> str:
    return "fsdp_params_gather_" + "_".join(str(i) for i in ids)


def padded_shard_numel(shape: Sequence[int], world_size: int) -> int:
    return math.ceil(shape[0] / world_size) * math.prod(shape[1:])


class ParamGroup:
    """One FSDP2 parameter group in the symmetric arena, as seen by the calling rank."""

    def __init__(self, shapes, dtype: torch.dtype, pg, param_dtype: Optional[torch.dtype] = None,
                 reduce_dtype: Optional[torch.dtype] = None, reduce_op: str = "avg", name: str = ""):
        self.shapes = [tuple(s) for s in shapes]
        self.dtype = dtype              # dtype of the sharded parameters (orig dtype)
        self.param_dtype = param_dtype  # dtype the unsharded parameters are used in (None = dtype)
        self.reduce_dtype = reduce_dtype
        self.reduce_op = reduce_op
        self.pg = pg
        self.world_size = group_size(pg)
        self.name = name
        W = self.world_size
        self.shard_numels = [padded_shard_numel(s, W) for s in self.shapes]
        self.offsets = [0]
        for n in self.shard_numels:
            self.offsets.append(self.offsets[-1] + n)
        self.total_shard_numel = self.offsets.pop()
        self.key = get_fsdp_params_key([id(self)] + list(range(len(self.shapes))))
        self.symm_buffer = SymmBufferRegistry.get_instance().get_or_create_symm_buffer(
            self.key, (self.total_shard_numel,), dtype
        )
        self._unsharded: Optional[List[torch.Tensor]] = None
        self._reduced = False

    # -- sharded parameters ---------------------------------------------------------------
    def local_shard_rows(self, p: int, rank: int) -> int:
        rows = math.ceil(self.shapes[p][0] / self.world_size)
        return max(0, min(rows, self.shapes[p][0] - rank * rows))

    def sharded_params(self, rank: Optional[int] = None) -> List[torch.Tensor]:
        """Rank's unpadded local shards as views of the symmetric buffer (fsdp2.py:187-196)."""
        rank = get_rank() if rank is None else rank
        buf = SymmBufferRegistry.get_instance().peer_tensors[self.key][rank]
        out = []
        for p, shape in enumerate(self.shapes):
            rows = self.local_shard_rows(p, rank)
            rest = math.prod(shape[1:])
            out.append(buf[self.offsets[p] : self.offsets[p] + rows * rest].view(rows, *shape[1:]))
        return out

    def load_full_params(self, params: Sequence[torch.Tensor]) -> None:
        """Shard full parameters over all W ranks' buffers (each rank copies its own chunk in
        the reference, fsdp2.py:186)."""
        peers = SymmBufferRegistry.get_instance().peer_tensors[self.key]
        for r in range(self.world_size):
            peers[r].zero_()
            for p, full in enumerate(params):
                assert tuple(full.shape) == self.shapes[p]
                rows = math.ceil(full.shape[0] / self.world_size)
                chunk = full[r * rows : (r + 1) * rows].reshape(-1).to(self.dtype)
                peers[r][self.offsets[p] : self.offsets[p] + chunk.numel()].copy_(chunk)

    # -- unshard ----------------------------------------------------------------------------
    def unshard(self, fused: bool = True) -> List[torch.Tensor]:
        W = self.world_size
        device = self.symm_buffer.device
        out_dtype = self.param_dtype or self.dtype
        gather = get_gather_service()
        if fused:
            # straight into per-parameter buffers, converted to the compute dtype on the way
            padded = [torch.empty(W * n, dtype=out_dtype, device=device) for n in self.shard_numels]
            gather.gather_slices(padded, self.symm_buffer, self.offsets, self.shard_numels, self.pg)
        else:
            padded = [torch.empty(W * n, dtype=self.dtype, device=device) for n in self.shard_numels]
            ag = torch.empty(W * self.total_shard_numel, dtype=self.dtype, device=device)
            gather.gather_into_tensor(ag, self.symm_buffer, self.pg)
            torch.split_with_sizes_copy(
                ag.view(W, -1), self.shard_numels, dim=1, out=[t.view(W, -1) for t in padded]
            )
            if out_dtype != self.dtype:
                padded = [t.to(out_dtype) for t in padded]  # fsdp2.py:341-343
        self._unsharded = [
            t.view(-1, *shape[1:])[: shape[0]] for t, shape in zip(padded, self.shapes)
        ]
        return self._unsharded

    def reshard(self) -> None:
        self._unsharded = None

    # -- reduce -----------------------------------------------------------------------------
    def reduce(self, unsharded_grads: Sequence[torch.Tensor], fused: bool = True) -> None:
        W = self.world_size
        scatter = get_reduction_service()
        grad_dtype = unsharded_grads[0].dtype
        reduce_dtype = self.reduce_dtype or grad_dtype
        for g, shape in zip(unsharded_grads, self.shapes):
            assert tuple(g.shape) == shape and g.dtype == grad_dtype
        if fused:
            scatter.scatter_accumulate_slices(
                id(self),
                [g.contiguous().view(-1) for g in unsharded_grads],
                self.offsets,
                self.shard_numels,
                self.pg,
                accumulation_numel=self.total_shard_numel,
                accumulation_dtype=reduce_dtype,
            )
        else:
            rs_input = torch.empty(
                W * self.total_shard_numel, dtype=reduce_dtype, device=unsharded_grads[0].device
            )
            torch._chunk_cat(list(unsharded_grads), dim=0, num_chunks=W, out=rs_input.view(W, -1))
            if id(self) not in scatter.accumulation_indices:
                scatter.register(id(self), (self.total_shard_numel,), reduce_dtype, reduce_dtype, self.pg)
            scatter.scatter_accumulate(id(self), rs_input, self.pg)
        self._reduced = True

    # -- publish ----------------------------------------------------------------------------
    def update_gradients(self) -> Optional[List[torch.Tensor]]:
        """fsdp2.py:836-847,897-939: average in place, cast to the parameter dtype, hand out the
        calling rank's sharded gradients as strided views of the accumulation."""
        if not self._reduced:
            return None  # no microbatch touched this group in this minibatch (fsdp2.py:797-801)
        self._reduced = False
        divisor = float(self.world_size) if self.reduce_op == "avg" else 1.0
        (reduce_output,) = get_reduction_service().publish(
            [id(self)], out_dtype=self.dtype, divisor=divisor
        )
        rank = get_rank()
        grads = []
        for p, shape in enumerate(self.shapes):
            rows = self.local_shard_rows(p, rank)
            size = (rows, *shape[1:])
            inner, acc = [], 1  # contiguous strides of (rows, *rest), valid for rows == 0 too
            for d in reversed(shape[1:]):
                inner.append(acc)
                acc *= d
            stride = (acc, *reversed(inner))
            grads.append(
                torch.as_strided(
                    reduce_output, size=size, stride=stride,
                    storage_offset=reduce_output.storage_offset() + self.offsets[p],
                )
            )
        self.sharded_grads = grads
        return grads


def _param_groups(fsdp_module) -> List[ParamGroup]:
    groups = getattr(fsdp_module, "_odc_param_groups", None)
    if groups is None:
        raise NotImplementedError(
            "expected an object with `_odc_param_groups` (a list of ParamGroup); rewiring a real "
            "torch fully_shard module needs a process group of W real ranks and is not done here"
        )
    return list(groups)


def pre_minibatch_start(fsdp_module):
    """fsdp2.py:427-433 (without the HPZ reshard)."""
    get_reduction_service().clear_accumulations()
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        torch.distributed.barrier()


def pre_optimizer_step(fsdp_module):
    """fsdp2.py:1023-1046: sync once, then publish every group's gradients."""
    scatter = get_reduction_service()
    for i, group in enumerate(_param_groups(fsdp_module)):
        if i == 0:
            with torch.cuda.nvtx.range("scatter_accumulate_sync"):
                scatter.sync(group.pg)
        with torch.cuda.nvtx.range(f"update_gradients:{group.name}"):
            group.update_gradients()


def patch_fsdp2(enable_hpz: bool = False) -> None:
    """Create the two services (fsdp2.py:1135-1138)."""
    global _enable_hpz, reduction_service, gather_service
    if enable_hpz:
        raise NotImplementedError("HPZ needs more than one node; not part of this build")
    _enable_hpz = False
    reduction_service = ReductionService()
    gather_service = GatherService()


def stop():
    get_reduction_service().stop()
    SymmBufferRegistry.get_instance().finalize()
    finalize_distributed()


def get_symm_buffer_memory_breakdown() -> dict:
    """Symmetric memory per rank in GB by key prefix (fsdp2.py:1147-1172)."""
    breakdown = {k: 0 for k in ("fsdp_params", "accumulation", "shared_buffer", "ag_buffer", "hpz_buffer", "other")}
    prefixes = (("fsdp_params_gather_", "fsdp_params"), ("rs_accumulation_", "accumulation"),
                ("shared_buffer_", "shared_buffer"), ("ag_buffer_", "ag_buffer"), ("hpz_", "hpz_buffer"))
    for key, tensor in SymmBufferRegistry.get_instance().local_tensor.items():
        for prefix, name in prefixes:
            if str(key).startswith(prefix):
                breakdown[name] += tensor.nbytes
                break
        else:
            breakdown["other"] += tensor.nbytes
    return {k: round(v / (1024**3), 2) for k, v in breakdown.items()}
