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

The same data flow is wired into torch's own ``fully_shard`` modules by ``patch_fsdp2`` +
``patch_lazy_init`` (fsdp2.py:103-112, 1105-1138): torch's ``foreach_all_gather``,
``foreach_all_gather_copy_out`` and ``foreach_reduce`` are replaced with versions that gather the
group's symmetric buffer straight into the parameters' unsharded storage (dtype conversion fused)
and scatter-accumulate the unsharded gradients straight into the group's accumulation; gradients
are handed to the sharded parameters at ``pre_optimizer_step``. One process plays one rank of a W
rank mesh (for instance over torch's "fake" process-group backend); the other ranks' shards are
passive memory, filled with ``fill_peer_shards``.

HPZ (fsdp2.py:551-582, 745-791, 961-1099) and the HSDP all-reduce (fsdp2.py:849-885) need more
than one node and are not part of this build.
"""

from __future__ import annotations

import logging
import math
import os
from typing import List, Optional, Sequence

import torch

from odc_amd.fsdp.shard_copies import compute_dtype_shards_of, shards_may_have_changed
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
_compute_dtype_shards = False  # patch_fsdp2(compute_dtype_shards=...)


def get_reduction_service():
    return reduction_service


def get_gather_service():
    return gather_service


class _GatherWork:
    """What ``ODCAllGather`` returns for ``async_op=True``: torch calls ``wait()`` on it before
    the copy-out. The gather was launched on the caller's stream, so the wait is an event."""

    def __init__(self):
        self.event = torch.cuda.Event()
        self.event.record()

    def wait(self, timeout=None):
        torch.cuda.current_stream().wait_event(self.event)
        return True


def _make_odc_all_gather():
    from torch.distributed.fsdp._fully_shard._fsdp_collectives import AllGather, DefaultAllocMixin

    class ODCAllGather(DefaultAllocMixin, AllGather):
        """torch's pluggable all-gather (``FSDPModule.set_custom_all_gather``) over the gather
        primitive, for group buffers that live in the symmetric arena: the reference's class of
        the same name (fsdp2.py:76-90). ``patch_fsdp2`` does not need it (its ``foreach_all_gather``
        gathers straight into the parameters); it serves code that keeps torch's copy-in /
        copy-out and only swaps the collective, and ``input_tensor`` must then be symmetric."""

        def __call__(self, output_tensor, input_tensor, group, async_op=False):
            get_gather_service().gather_into_tensor(output_tensor, input_tensor, group)
            return _GatherWork() if async_op else None

    return ODCAllGather


_odc_gather_comm = None


def get_odc_gather_comm():
    """The process-wide ``ODCAllGather`` (fsdp2.py:208-212)."""
    global _odc_gather_comm
    if _odc_gather_comm is None:
        _odc_gather_comm = _make_odc_all_gather()()
    return _odc_gather_comm


def get_fsdp_params_key(ids: Sequence[int]) -> str:
    return "fsdp_params_gather_" + "_".join(str(i) for i in ids)


def padded_shard_numel(shape: Sequence[int], world_size: int) -> int:
    return math.ceil(shape[0] / world_size) * math.prod(shape[1:])


# The kernels work in tiles of 4096 elements, and the read-modify-write of the scatter-accumulate
# streams 3 % faster when its tiles start on tile-sized boundaries of the accumulation (16 KiB of
# fp32; measured on a Llama-3-8B layer). The group's accumulation is private to this module (the
# sharded gradients are handed out as views), so its slices need not be packed the way the
# reduce-scatter output of the reference is: every slice of a tile or more starts on a tile.
ACCUMULATION_SLICE_ALIGN = 4096


def tile_aligned_offsets(numels: Sequence[int], align: int = ACCUMULATION_SLICE_ALIGN):
    """``(offsets, total)`` of slices of ``numels`` elements laid out in order, each slice of at
    least ``align`` elements starting on a multiple of ``align``."""
    offsets, end = [], 0
    for n in numels:
        if n >= align:
            end = -(-end // align) * align
        offsets.append(end)
        end += n
    return offsets, end


class ParamGroup:
    """One FSDP2 parameter group in the symmetric arena, as seen by the calling rank."""

    def __init__(self, shapes, dtype: torch.dtype, pg, param_dtype: Optional[torch.dtype] = None,
                 reduce_dtype: Optional[torch.dtype] = None, reduce_op: str = "avg", name: str = "",
                 compute_dtype_shards: bool = False):
        self.shapes = [tuple(s) for s in shapes]
        # keep a copy of the shards in param_dtype and gather from it (compute_dtype_shards_of)
        self.compute_dtype_shards = compute_dtype_shards
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
        # where the slices lie in the accumulation: packed like the shards when the two-step
        # (reference) flow fills it with one flat reduce-scatter input, tile aligned when the
        # fused flow does; fixed by the first reduce
        self.acc_offsets: Optional[List[int]] = None
        self._aligned_acc_layout = tile_aligned_offsets(self.shard_numels)
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
        shards_may_have_changed()

    # -- unshard ----------------------------------------------------------------------------
    def unshard(self, fused: bool = True) -> List[torch.Tensor]:
        W = self.world_size
        device = self.symm_buffer.device
        out_dtype = self.param_dtype or self.dtype
        gather = get_gather_service()
        if fused:
            # straight into per-parameter buffers, converted to the compute dtype on the way
            padded = [torch.empty(W * n, dtype=out_dtype, device=device) for n in self.shard_numels]
            source = self.symm_buffer
            if self.compute_dtype_shards and out_dtype != self.dtype:
                # the shards handed out by sharded_params() are views of the symmetric buffer and
                # share its version counter: writes through them are seen without a watch list
                source = compute_dtype_shards_of(gather, self.key, self.total_shard_numel, out_dtype)
            gather.gather_slices(padded, source, self.offsets, self.shard_numels, self.pg)
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
        acc_offsets, acc_total = self._aligned_acc_layout if fused else (self.offsets, self.total_shard_numel)
        if self.acc_offsets is None:
            self.acc_offsets = acc_offsets
        elif self.acc_offsets != acc_offsets:
            raise RuntimeError("a parameter group reduces either fused or in two steps, not both: "
                               "the two flows lay the accumulation out differently")
        if fused:
            scatter.scatter_accumulate_slices(
                id(self),
                [g.contiguous().view(-1) for g in unsharded_grads],
                acc_offsets,
                self.shard_numels,
                self.pg,
                accumulation_numel=acc_total,
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
        # the gradients are handed out as views of the slices: nothing is written between them
        (reduce_output,) = get_reduction_service().publish(
            [id(self)], out_dtype=self.dtype, divisor=divisor, within_slices=True
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
                    storage_offset=reduce_output.storage_offset() + self.acc_offsets[p],
                )
            )
        self.sharded_grads = grads
        return grads


# ------------------------------------------------------------------------------------------------
# torch fully_shard integration
# ------------------------------------------------------------------------------------------------
def _torch_param_groups(fsdp_module):
    """All FSDPParamGroups under a ``fully_shard`` root module (fsdp2.py:1026-1030)."""
    from torch.distributed.fsdp import fully_shard

    root_state = fully_shard.state(fsdp_module)
    root_state._lazy_init()
    return [
        st._fsdp_param_group for st in root_state._state_ctx.all_states if st._fsdp_param_group is not None
    ]


def _group_layout(fsdp_param_group):
    return fsdp_param_group._odc_layout


class _GroupLayout:
    """Where each FSDPParam of a torch param group lives in the group's symmetric buffer."""

    def __init__(self, fsdp_param_group):
        params = fsdp_param_group.fsdp_params
        self.key = get_fsdp_params_key([id(p) for p in params])
        self.dtype = params[0]._sharded_param_data.dtype
        for fp in params:
            if fp._sharded_param_data.dtype != self.dtype:
                raise ValueError(
                    f"All FSDP parameters must have the same dtype: {fp._sharded_param_data.dtype=} {self.dtype=}"
                )
            if fp.fsdp_placement.dim != 0:
                raise NotImplementedError("only dim-0 sharding is wired to the fused kernels")
        self.numels = [fp._sharded_param_data.numel() for fp in params]
        self.offsets = [0]
        for n in self.numels:
            self.offsets.append(self.offsets[-1] + n)
        self.total = self.offsets.pop()
        # the group's accumulation: the same slices, tile aligned
        self.acc_offsets, self.acc_total = tile_aligned_offsets(self.numels)
        self.index = {id(fp): i for i, fp in enumerate(params)}


@torch.no_grad()
def replace_sharded_param_with_symm_buffer(fsdp_model) -> None:
    """Move the group's sharded parameters into one symmetric buffer and point the FSDPParams
    (and their DTensors' local tensors) at views of it (fsdp2.py:116-202, without HPZ)."""
    if _enable_hpz is None:
        raise ValueError("Need to run patch_fsdp2() first")
    group = fsdp_model._get_fsdp_state()._fsdp_param_group
    if group is None or hasattr(group, "_odc_layout"):
        return
    layout = _GroupLayout(group)
    symm_buffer = SymmBufferRegistry.get_instance().get_or_create_symm_buffer(
        layout.key, (layout.total,), layout.dtype
    )
    for fp, off, n in zip(group.fsdp_params, layout.offsets, layout.numels):
        assert math.prod(fp.padded_sharded_param_size) == n
        piece = symm_buffer[off : off + n]
        piece.copy_(fp._sharded_param_data)
        padded = piece.view(fp.padded_sharded_param_size)
        fp._sharded_param_data = padded.view(-1)
        old_local = fp.sharded_param._local_tensor
        length = old_local.size(0) if old_local.numel() > 0 else 0
        fp.sharded_param._local_tensor = padded.narrow(dim=0, start=0, length=length)
        fp._odc_group = group
    group._odc_layout = layout
    group._odc_symm_buffer = symm_buffer
    # a checkpoint load rewrites the shards: copies kept in the compute dtype are made anew
    fsdp_model.register_load_state_dict_post_hook(_after_load_state_dict)


def _after_load_state_dict(module, incompatible_keys) -> None:
    shards_may_have_changed()


@torch.no_grad()
def patch_lazy_init(fsdp_model) -> None:
    """Run ``replace_sharded_param_with_symm_buffer`` right after the group's own lazy init
    (fsdp2.py:103-112)."""
    import types

    group = fsdp_model._get_fsdp_state()._fsdp_param_group
    if group is None:
        return
    prev_lazy_init = group.lazy_init

    def patched_lazy_init(_self):
        prev_lazy_init()
        replace_sharded_param_with_symm_buffer(fsdp_model)

    group.lazy_init = types.MethodType(patched_lazy_init, group)


@torch.no_grad()
def fill_peer_shards(fsdp_model, full_params) -> None:
    """Virtual-world helper: write rank r's chunk of every full parameter into rank r's region,
    for all r (in the reference every process does this for itself at lazy init).
    ``full_params`` maps a parameter's fully qualified name (as the root module names it) to
    the full, unsharded tensor."""
    group = fsdp_model._get_fsdp_state()._fsdp_param_group
    if group is None:
        return
    layout = _group_layout(group)
    peers = SymmBufferRegistry.get_instance().peer_tensors[layout.key]
    W = len(peers)
    for fp, off, n in zip(group.fsdp_params, layout.offsets, layout.numels):
        full = full_params[fp._param_fqn]
        rows = math.ceil(full.shape[0] / W)
        for r in range(W):
            chunk = full[r * rows : (r + 1) * rows].reshape(-1).to(layout.dtype)
            peers[r][off : off + n].zero_()
            peers[r][off : off + chunk.numel()].copy_(chunk)
    shards_may_have_changed()


@torch.no_grad()
def foreach_all_gather(fsdp_params, group, async_op, all_gather_copy_in_stream, all_gather_stream,
                       device, all_gather_comm):
    """Replacement for torch's ``foreach_all_gather`` (fsdp2.py:219-313): no copy-in, no
    intermediate ``[W, sum n_p]`` buffer — the group's symmetric buffer is gathered straight into
    every parameter's unsharded storage, converted to ``param_dtype`` on the way."""
    from torch.distributed.device_mesh import _get_device_handle
    from torch.distributed.fsdp._fully_shard._fsdp_collectives import AllGatherResult

    fsdp_group = fsdp_params[0]._odc_group
    layout = _group_layout(fsdp_group)
    world_size = group.size()
    device_handle = _get_device_handle(device.type)
    out_dtype = fsdp_params[0].param_dtype or layout.dtype
    outs, offsets, numels, dtypes_meta, numels_meta = [], [], [], [], []
    consumer_stream = device_handle.current_stream()
    all_gather_stream.wait_stream(all_gather_copy_in_stream)
    with device_handle.stream(all_gather_stream):
        # The unsharded storages are written here, on a stream that runs ahead of the consumer
        # (implicit prefetch), so they must come from THIS stream's pool: a block of the
        # consumer's pool may still be in use by kernels queued there. record_stream hands the
        # block back only after the consumer's work queued up to the free has finished.
        for fp in fsdp_params:
            i = layout.index[id(fp)]
            n = layout.numels[i]
            fp.init_all_gather_outputs([n], [out_dtype], world_size, device)
            fp.alloc_all_gather_outputs()
            out = fp.all_gather_outputs[0]
            if consumer_stream != all_gather_stream:
                out.record_stream(consumer_stream)
            outs.append(out)
            offsets.append(layout.offsets[i])
            numels.append(n)
            dtypes_meta.append([out_dtype])
            numels_meta.append([n])
        source = fsdp_group._odc_symm_buffer
        if _compute_dtype_shards and out_dtype != layout.dtype:
            source = compute_dtype_shards_of(get_gather_service(), layout.key, layout.total, out_dtype,
                                             watch=[fp.sharded_param for fp in fsdp_group.fsdp_params])
        get_gather_service().gather_slices(outs, source, offsets, numels, group)
        all_gather_event = all_gather_stream.record_event()
    placeholder = torch.empty(0, dtype=out_dtype, device=device)
    return AllGatherResult(placeholder, all_gather_event, None, dtypes_meta, numels_meta, numels)


@torch.no_grad()
def foreach_all_gather_copy_out(all_gather_result, fsdp_params, group) -> None:
    """The copy-out already happened inside the gather; only the stream dependency is left
    (fsdp2.py:317-424)."""
    event = all_gather_result.all_gather_event
    if event is not None:
        torch.cuda.current_stream().wait_event(event)


@torch.no_grad()
def foreach_reduce(fsdp_params, unsharded_grads, reduce_scatter_group, reduce_scatter_stream,
                   reduce_scatter_comm, orig_dtype, reduce_dtype, device, gradient_divide_factor,
                   all_reduce_group, all_reduce_stream, all_reduce_grads, partial_reduce_output,
                   all_reduce_hook, force_sum_reduction_for_comms=False):
    """Replacement for torch's ``foreach_reduce`` (fsdp2.py:608-742): the unsharded gradients are
    scatter-accumulated straight into the group's accumulation (zero padding and the cast to the
    reduce dtype happen in the kernel); handing gradients to the sharded parameters is deferred
    to ``pre_optimizer_step``."""
    from torch.distributed.device_mesh import _get_device_handle
    from torch.distributed.fsdp._fully_shard._fsdp_collectives import (
        _div_if_needed,
        _get_gradient_divide_factors,
    )

    if all_reduce_group is not None:
        raise NotImplementedError("HSDP needs more than one node; not part of this build")
    grad_dtypes = {g.dtype for g in unsharded_grads}
    if len(grad_dtypes) != 1:
        raise AssertionError(f"FSDP reduce-scatter expects uniform gradient dtype but got {grad_dtypes}")
    grad_dtype = unsharded_grads[0].dtype
    reduce_dtype = reduce_dtype or grad_dtype
    predivide_factor, _post, _rs_op, _ar_op = _get_gradient_divide_factors(
        reduce_scatter_group, all_reduce_group, reduce_dtype, device.type, gradient_divide_factor,
        force_sum_reduction_for_comms,
    )
    fsdp_group = fsdp_params[0]._odc_group
    layout = _group_layout(fsdp_group)
    device_handle = _get_device_handle(device.type)
    current_stream = device_handle.current_stream()
    reduce_scatter_stream.wait_stream(current_stream)
    with device_handle.stream(reduce_scatter_stream):
        grads, offsets, numels = [], [], []
        for fp, g in zip(fsdp_params, unsharded_grads):
            i = layout.index[id(fp)]
            g = g.contiguous().view(-1)
            if predivide_factor is not None and predivide_factor > 1 and g.dtype != reduce_dtype:
                # fp16 reduction of bf16/fp32 gradients: the reference divides AFTER the cast to
                # the reduce dtype (fsdp2.py:676-690); keep that order of roundings
                g = g.to(reduce_dtype)
            _div_if_needed(g, predivide_factor)
            g.record_stream(reduce_scatter_stream)  # read there after the caller drops its list
            grads.append(g)
            offsets.append(layout.acc_offsets[i])
            numels.append(layout.numels[i])
        get_reduction_service().scatter_accumulate_slices(
            id(fsdp_group), grads, offsets, numels, reduce_scatter_group,
            accumulation_numel=layout.acc_total, accumulation_dtype=reduce_dtype,
        )
        reduce_scatter_event = reduce_scatter_stream.record_event()
        # parameters that got a gradient in some microbatch of this minibatch: only they are
        # handed one at the optimizer step (frozen or unused parameters keep grad = None)
        touched = getattr(fsdp_group, "_odc_params_with_grad", None)
        if touched is None:
            touched = fsdp_group._odc_params_with_grad = set()
        touched.update(id(fp) for fp in fsdp_params)
        fsdp_group._odc_reduce_context = dict(
            reduce_scatter_group=reduce_scatter_group, reduce_scatter_stream=reduce_scatter_stream,
            orig_dtype=orig_dtype, reduce_dtype=reduce_dtype, device=device,
            gradient_divide_factor=gradient_divide_factor, all_reduce_hook=all_reduce_hook,
            force_sum_reduction_for_comms=force_sum_reduction_for_comms, grad_dtype=grad_dtype,
        )
        post_reduce_event = reduce_scatter_stream.record_event()
    unsharded_grads.clear()
    placeholder = torch.empty(0, dtype=reduce_dtype, device=device)
    return placeholder, reduce_scatter_event, post_reduce_event, None, None, partial_reduce_output


def _publish_request(fsdp_param_group):
    """First half of ``update_gradients`` (fsdp2.py:795-899) for a torch param group: take the
    group's reduce context and say what the end-of-minibatch pass over its accumulation is, as
    ``(key, out_dtype, divisor, touched)``; None when no microbatch ran through the group in this
    minibatch (fsdp2.py:797-801). Whatever cannot be folded into one pass (an all-reduce hook, a
    separate post-divide: two roundings) is done here."""
    import torch.distributed as dist
    from torch.distributed.fsdp._fully_shard._fsdp_collectives import _get_gradient_divide_factors

    ctx = getattr(fsdp_param_group, "_odc_reduce_context", None)
    if ctx is None:
        return None
    del fsdp_param_group._odc_reduce_context
    touched = fsdp_param_group.__dict__.pop("_odc_params_with_grad", None)
    rs_group = ctx["reduce_scatter_group"]
    _pre, postdivide_factor, reduce_scatter_op, _ar_op = _get_gradient_divide_factors(
        rs_group, None, ctx["reduce_dtype"], ctx["device"].type, ctx["gradient_divide_factor"],
        ctx["force_sum_reduction_for_comms"],
    )
    assert reduce_scatter_op in (dist.ReduceOp.SUM, dist.ReduceOp.AVG), f"{reduce_scatter_op} is not supported"
    scatter = get_reduction_service()
    key = id(fsdp_param_group)
    orig_dtype = ctx["orig_dtype"] or scatter.accumulation_dtype_of(key)
    if ctx["all_reduce_hook"] is not None or (postdivide_factor is not None and postdivide_factor > 1):
        # two roundings (average, then post-divide) and a user hook in between
        if reduce_scatter_op == dist.ReduceOp.AVG:
            scatter.publish([key], divisor=float(rs_group.size()), within_slices=ctx["all_reduce_hook"] is None)
        if ctx["all_reduce_hook"] is not None:
            ctx["all_reduce_hook"](scatter.get_accumulation(key))
        divisor = postdivide_factor if postdivide_factor is not None and postdivide_factor > 1 else 1.0
    else:
        divisor = float(rs_group.size()) if reduce_scatter_op == dist.ReduceOp.AVG else 1.0
    return key, orig_dtype, float(divisor), touched


def _hand_out_gradients(fsdp_param_group, reduce_output, touched) -> None:
    """Second half of ``update_gradients`` (fsdp2.py:902-939): strided views of the published
    shard become the sharded parameters' DTensor gradients."""
    from torch.distributed.tensor import DTensor

    layout = _group_layout(fsdp_param_group)
    base = reduce_output.storage_offset()
    for fp, off in zip(fsdp_param_group.fsdp_params, layout.acc_offsets):
        if touched is not None and id(fp) not in touched:
            continue
        new_sharded_grad = torch.as_strided(
            reduce_output, size=fp.sharded_size, stride=fp.contiguous_sharded_stride,
            storage_offset=base + off,
        )
        if fp.sharded_param.grad is not None:
            assert isinstance(fp.sharded_param.grad, DTensor)
            fp.sharded_param.grad._local_tensor += new_sharded_grad
        else:
            fp.sharded_param.grad = fp.to_sharded_dtensor(new_sharded_grad)
        for hook in (getattr(fp.sharded_param, "_post_accumulate_grad_hooks", {}) or {}).values():
            hook(fp.sharded_param)


@torch.no_grad()
def update_gradients(fsdp_param_group) -> None:
    """fsdp2.py:795-957 for one torch param group: average and post-divide the calling rank's
    accumulation in place, cast to the parameter dtype, hand the strided views to the sharded
    parameters as DTensor gradients."""
    request = _publish_request(fsdp_param_group)
    if request is None:
        return
    key, out_dtype, divisor, touched = request
    (reduce_output,) = get_reduction_service().publish([key], out_dtype=out_dtype, divisor=divisor,
                                                       within_slices=True)
    _hand_out_gradients(fsdp_param_group, reduce_output, touched)


@torch.no_grad()
def update_all_gradients(fsdp_param_groups) -> None:
    """``update_gradients`` for every group of a model with as few passes as possible: the
    groups whose accumulations share (accumulation dtype, gradient dtype, divisor) are divided
    and cast by ONE launch (per 64 groups) instead of one short launch each."""
    scatter = get_reduction_service()
    batches = {}
    for group in fsdp_param_groups:
        request = _publish_request(group)
        if request is None:
            continue
        key, out_dtype, divisor, touched = request
        batches.setdefault((scatter.accumulation_dtype_of(key), out_dtype, divisor), []).append((group, key, touched))
    for (_acc_dtype, out_dtype, divisor), members in batches.items():
        outputs = scatter.publish([key for _, key, _ in members], out_dtype=out_dtype, divisor=divisor,
                                  within_slices=True)
        for (group, _key, touched), reduce_output in zip(members, outputs):
            with torch.cuda.nvtx.range(f"update_gradients:{group._module_fqn}"):
                _hand_out_gradients(group, reduce_output, touched)


def _is_torch_fsdp_module(fsdp_module) -> bool:
    return hasattr(fsdp_module, "_get_fsdp_state")


def _param_groups(fsdp_module) -> List[ParamGroup]:
    groups = getattr(fsdp_module, "_odc_param_groups", None)
    if groups is None:
        raise TypeError("expected a fully_shard module or an object with `_odc_param_groups`")
    return list(groups)


def pre_minibatch_start(fsdp_module):
    """fsdp2.py:427-433 (without the HPZ reshard)."""
    shards_may_have_changed()  # copies of the shards in the compute dtype are made anew
    get_reduction_service().clear_accumulations()
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        torch.distributed.barrier()


def pre_optimizer_step(fsdp_module):
    """fsdp2.py:1023-1046: sync once, then publish every group's gradients."""
    shards_may_have_changed()  # the optimizer is about to change the shards
    scatter = get_reduction_service()
    if _is_torch_fsdp_module(fsdp_module):
        groups = _torch_param_groups(fsdp_module)
        if groups:
            with torch.cuda.nvtx.range("scatter_accumulate_sync"):
                scatter.sync(groups[0].mesh_info.shard_process_group)
            update_all_gradients(groups)
        return
    for i, group in enumerate(_param_groups(fsdp_module)):
        if i == 0:
            with torch.cuda.nvtx.range("scatter_accumulate_sync"):
                scatter.sync(group.pg)
        with torch.cuda.nvtx.range(f"update_gradients:{group.name}"):
            group.update_gradients()


def _comm_context_lazy_init(self, device):
    """``FSDPCommContext.lazy_init`` with the all-gather and reduce-scatter streams at the default
    priority, always. torch creates them at high priority so that its copy-in / copy-out kernels
    are not delayed behind compute; the launches here gain nothing from it on MI355X (Llama
    example: 21.8 ms per microbatch with default-priority streams, 21.7 with torch's), and work
    queued on streams of different priorities is a hazard on this platform (it has hung) and
    costly (with the launches on the reference's dedicated comm stream next to torch's
    high-priority streams the same microbatch took 28.2 ms, with all streams at the default
    priority 21.6). So there is no switch that keeps torch's priorities."""
    from torch.distributed.fsdp._fully_shard import _fsdp_param_group

    _fsdp_param_group.FSDPCommContext._odc_original_lazy_init(self, device)
    self.all_gather_copy_in_stream = self.device_handle.Stream()
    self.all_gather_stream = self.device_handle.Stream()
    self.reduce_scatter_stream = self.device_handle.Stream()


_RECORD_FUNCTION_HOMES = ("torch.distributed.fsdp._fully_shard._fsdp_param_group", "torch.profiler",
                          "torch.autograd.profiler")
_original_record_functions = {}


def _forward_record_function_to_markers() -> None:
    """torch's ``record_function`` ranges (FSDP brackets unshard, reshard, the hooks and the
    reductions with them) also as marker ranges, so that a ``rocprofv3 --marker-trace`` timeline
    shows them around the primitive launches: the reference's ``nvtx_record_function``, installed
    in the same three places (fsdp2.py:54-61, 1131-1133). Here only under ``ODC_TRACE=1``, the
    switch of the primitives' own marker ranges; ``unpatch_fsdp2`` puts torch's class back."""
    import importlib

    from torch.autograd.profiler import record_function

    if _original_record_functions:
        return

    class marker_record_function(record_function):
        def __enter__(self):
            torch.cuda.nvtx.range_push(self.name)
            return super().__enter__()

        def __exit__(self, exc_type, exc_value, traceback):
            try:
                return super().__exit__(exc_type, exc_value, traceback)
            finally:
                torch.cuda.nvtx.range_pop()

    for home in _RECORD_FUNCTION_HOMES:
        module = importlib.import_module(home)
        _original_record_functions[home] = module.record_function
        module.record_function = marker_record_function


def _restore_record_function() -> None:
    import importlib

    for home, original in _original_record_functions.items():
        importlib.import_module(home).record_function = original
    _original_record_functions.clear()


def patch_fsdp2(enable_hpz: bool = False, compute_dtype_shards: Optional[bool] = None) -> None:
    """Create the two services and route torch's fully_shard collectives through them
    (fsdp2.py:1105-1138). Modules sharded afterwards need ``patch_lazy_init(module)`` each.

    ``compute_dtype_shards`` (default: ``$ODC_FSDP2_COMPUTE_DTYPE_SHARDS == "1"``, off): under a
    mixed-precision policy, keep every group's shards a second time in ``param_dtype`` and gather
    from that copy (``compute_dtype_shards_of``)."""
    global _enable_hpz, reduction_service, gather_service, _compute_dtype_shards
    if enable_hpz:
        raise NotImplementedError("HPZ needs more than one node; not part of this build")
    _enable_hpz = False
    if compute_dtype_shards is None:
        compute_dtype_shards = os.environ.get("ODC_FSDP2_COMPUTE_DTYPE_SHARDS", "0") == "1"
    _compute_dtype_shards = bool(compute_dtype_shards)
    from torch.distributed.fsdp._fully_shard import _fsdp_collectives, _fsdp_param_group

    comm_context = _fsdp_param_group.FSDPCommContext
    if not hasattr(comm_context, "_odc_original_lazy_init"):
        comm_context._odc_original_lazy_init = comm_context.lazy_init
        comm_context.lazy_init = _comm_context_lazy_init
    for module in (_fsdp_collectives, _fsdp_param_group):
        if not hasattr(module, "_odc_original_collectives"):
            module._odc_original_collectives = (
                module.foreach_all_gather, module.foreach_all_gather_copy_out, module.foreach_reduce,
            )
        module.foreach_all_gather = foreach_all_gather
        module.foreach_all_gather_copy_out = foreach_all_gather_copy_out
        module.foreach_reduce = foreach_reduce
    if os.environ.get("ODC_TRACE", "0") == "1":
        _forward_record_function_to_markers()
    reduction_service = ReductionService()
    gather_service = GatherService()


def unpatch_fsdp2() -> None:
    """Put torch's own collectives back (for running patched and unpatched in one process)."""
    from torch.distributed.fsdp._fully_shard import _fsdp_collectives, _fsdp_param_group

    for module in (_fsdp_collectives, _fsdp_param_group):
        orig = getattr(module, "_odc_original_collectives", None)
        if orig is not None:
            module.foreach_all_gather, module.foreach_all_gather_copy_out, module.foreach_reduce = orig
            del module._odc_original_collectives
    comm_context = _fsdp_param_group.FSDPCommContext
    if hasattr(comm_context, "_odc_original_lazy_init"):
        comm_context.lazy_init = comm_context._odc_original_lazy_init
        del comm_context._odc_original_lazy_init
    _restore_record_function()


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
