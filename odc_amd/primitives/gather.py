"""On-demand gather: W sharded buffers -> one full flat buffer, one fused HIP launch.

Mirror of ``odc/primitives/gather.py`` (``GatherService.gather_into_tensor``, :76-127,176). The
reference issues W peer ``copy_``s on a side stream; here the same result comes from
``odc_gather`` (include/odc_hip.h), whose work list covers all W shards of all tensors of the
call. The inter-node NVSHMEM branch of the reference (:129-175) has no counterpart on one GPU.
"""

from __future__ import annotations

import ctypes
import logging
import threading
from typing import Sequence

import torch
from torch import Tensor

from odc_amd import _native
from odc_amd.primitives.utils import (
    BufferSplitter,
    SymmBufferRegistry,
    comm_stream_section,
    get_rank,
    get_world,
    group_size,
    native_dtype,
    stream_from_handle,
)

logger = logging.getLogger(__name__)


class _GatherPlan:
    """The cached part of one gather call: its item array with everything but the output
    pointers filled in."""

    __slots__ = ("items", "n", "cast", "src_code", "dst_code", "out_numels")


class GatherService:
    def __init__(self):
        self.buffer_splitter = BufferSplitter()
        self._plans = threading.local()  # per host thread: plan key -> _GatherPlan
        self._lock = threading.Lock()
        self._conversion = None  # (stream handle, event) of the latest convert_symm_buffer
        self._met_conversion = frozenset()  # streams ordered after it (replaced, never mutated)

    def gather_into_tensor(self, output_tensor: Tensor, input_tensor: Tensor, pg) -> None:
        """``output_tensor.view(W, -1)[r] = rank r's copy of input_tensor`` for every r.

        ``input_tensor`` is the calling rank's shard and must live in a registered symmetric
        buffer; ``pg`` is a process group or ``VirtualGroup`` of the arena's W ranks.
        """
        self.gather_into_tensors([output_tensor], [input_tensor], pg)

    def gather_into_tensors(
        self, output_tensors: Sequence[Tensor], input_tensors: Sequence[Tensor], pg
    ) -> None:
        """Multi-tensor form: every (output, input) pair of the lists in ONE launch (per 64
        pairs). Equivalent to calling ``gather_into_tensor`` pair by pair. When the outputs'
        dtype differs from the shards' (bf16/fp16/fp32 only) the conversion is fused in."""
        assert len(output_tensors) == len(input_tensors)
        world = get_world()  # raises when there is no arena (no GPU, or init_nvshmem not called)
        if not len(input_tensors):
            return
        src_dtype = input_tensors[0].dtype
        pointers, numels = [], []
        for inp in input_tensors:
            assert inp.is_cuda and inp.is_contiguous(), "shards are contiguous GPU tensors"
            assert inp.dtype == src_dtype, "one launch takes one dtype pair"
            pointers.append(inp.data_ptr())
            numels.append(inp.numel())
        # where a shard lies in the arena follows from its address alone, so the symmetric
        # offsets of a list of shards are looked up once per list of addresses (and host thread)
        cache = getattr(self._plans, "offsets", None)
        if cache is None:
            cache = self._plans.offsets = {}
        key = (world.serial, tuple(pointers), tuple(numels))
        known = cache.get(key)
        if known is None:
            registry = SymmBufferRegistry.get_instance()
            keep = [k for k, n in enumerate(numels) if n]
            known = cache[key] = (
                keep if len(keep) != len(numels) else None,
                [registry.symmetric_offset_of(input_tensors[k]) for k in keep],
                [numels[k] for k in keep],
            )
        keep, offsets, kept_numels = known
        if keep is not None:  # empty shards have empty outputs and take no part in the launch
            for k, n in enumerate(numels):
                assert n or not output_tensors[k].numel(), f"output {k} is not empty but its shard is"
            output_tensors = [output_tensors[k] for k in keep]
            if not output_tensors:
                return
        self._gather(output_tensors, offsets, kept_numels, src_dtype, pg)

    def _gather(self, outs, src_offsets, shard_numels, src_dtype, pg) -> None:
        """One launch (per 64 items): ``outs[k].view(W, -1)[r]`` = the ``shard_numels[k]`` elements
        of ``src_dtype`` at symmetric byte offset ``src_offsets[k]`` of rank r. The item array is
        built once per (offsets, sizes, dtypes) and host thread; later calls only rewrite the
        output pointers."""
        world = get_world()
        W = group_size(pg)
        assert W == world.world_size, f"group size {W} != arena world size {world.world_size}"
        dst_dtype = outs[0].dtype
        cache = getattr(self._plans, "cache", None)
        if cache is None:
            cache = self._plans.cache = {}
        plan_key = (world.serial, tuple(src_offsets), tuple(shard_numels), src_dtype, dst_dtype)
        plan = cache.get(plan_key)
        if plan is None:
            plan = cache[plan_key] = _GatherPlan()
            plan.n = len(outs)
            plan.cast = src_dtype != dst_dtype
            plan.items = ((_native.GatherCastItem if plan.cast else _native.GatherItem) * plan.n)()
            plan.out_numels = [W * n for n in shard_numels]
            es = src_dtype.itemsize
            for item, offset, n in zip(plan.items, src_offsets, shard_numels):
                item.src_offset = offset
                if plan.cast:
                    item.shard_elems = n
                else:
                    item.shard_bytes = n * es
            # shards kept in one dtype (fp32 master copies), full parameter wanted in another
            # (bf16): converted on the way instead of gathered and then cast
            # (odc/fsdp/fsdp1.py:199-223, odc/fsdp/fsdp2.py:341-343)
            plan.src_code = native_dtype(src_dtype) if plan.cast else None
            plan.dst_code = native_dtype(dst_dtype) if plan.cast else None
        items = plan.items
        for item, out, numel in zip(items, outs, plan.out_numels):
            assert out.is_cuda, "gather runs on the GPU only"
            assert out.dtype == dst_dtype, "one launch takes one dtype pair"
            assert out.is_contiguous()
            assert out.numel() == numel, f"output numel {out.numel()} != {W} * shard numel {numel // W}"
            item.dst = out.data_ptr()

        lib = _native.load()
        with comm_stream_section("odc.gather") as comm:
            if self._conversion is not None:
                self._order_after_conversion(comm.cuda_stream)
            stream = ctypes.c_void_p(comm.cuda_stream)
            if plan.cast:
                status = lib.odc_gather_cast(
                    world.arena.handle, items, plan.n, plan.src_code, plan.dst_code, get_rank(), stream
                )
            else:
                status = lib.odc_gather(world.arena.handle, items, plan.n, get_rank(), stream)
        if status:
            _native.check(status)

    def gather_slices(
        self,
        output_tensors: Sequence[Tensor],
        input_tensor: Tensor,
        slice_offsets: Sequence[int],
        slice_numels: Sequence[int],
        pg,
    ) -> None:
        """Gather slices of ONE symmetric buffer straight into separate outputs, in one launch:
        ``output_i.view(W, -1)[r] = rank r's input_tensor[off_i : off_i + n_i]``.

        With the FSDP2 group layout (``odc/fsdp/fsdp2.py:146-196``: the group buffer is the
        concatenation of every parameter's padded shard) this is ``gather_into_tensor`` followed
        by ``split_with_sizes_copy(dim=1)`` (``fsdp2.py:378-401``) without the intermediate
        ``[W, sum n_i]`` buffer.
        """
        assert len(output_tensors) == len(slice_offsets) == len(slice_numels)
        assert input_tensor.is_cuda and input_tensor.is_contiguous()
        if not len(output_tensors):
            return
        es = input_tensor.element_size()
        total = input_tensor.numel()
        base = SymmBufferRegistry.get_instance().symmetric_offset_of(input_tensor)
        outs, offsets, numels = [], [], []
        for out, off, n in zip(output_tensors, slice_offsets, slice_numels):
            assert 0 <= off and off + n <= total, "slice leaves the buffer"
            if n or out.numel():
                outs.append(out)
                offsets.append(base + off * es)
                numels.append(n)
        if outs:
            self._gather(outs, offsets, numels, input_tensor.dtype, pg)

    def convert_symm_buffer(self, dst_key, src_key, ranks: Sequence[int] = None) -> None:
        """Rank r's symmetric buffer ``dst_key`` = rank r's ``src_key`` converted to the
        destination's dtype (round to nearest even), for every rank whose memory this process
        holds, in ONE launch over all W regions (``odc_convert``); ``ranks`` narrows it to some
        ranks, one launch each (with one process per GPU a rank converts its own shard). On the
        launch stream of the other primitives; a gather issued later on another stream first
        waits for the conversion.

        It is what keeps a copy of the sharded parameters in the compute dtype: converted once
        after the optimizer step (4 + 2 bytes per element of ONE shard), so that every gather of
        the minibatch moves 2 + 2 bytes per element instead of converting on the way (4 + 2),
        the FSDP2 counterpart of the copy-once-until-flush of ``odc/primitives/utils.py:103-116``
        that ``odc/fsdp/fsdp1.py:239-247`` uses for the low-precision shard."""
        registry = SymmBufferRegistry.get_instance()
        world = get_world()
        src_offset, src_shape, src_dtype = registry.offsets[src_key]
        dst_offset, dst_shape, dst_dtype = registry.offsets[dst_key]
        assert tuple(src_shape) == tuple(dst_shape), f"{src_key}: {src_shape} != {dst_key}: {dst_shape}"
        numel = 1
        for d in src_shape:
            numel *= d
        if not numel:
            return
        lib = _native.load()
        with comm_stream_section("odc.convert") as comm:
            stream = ctypes.c_void_p(comm.cuda_stream)
            if ranks is None:
                item = (_native.ConvertItem * 1)()
                item[0].src_offset, item[0].dst_offset, item[0].elems = src_offset, dst_offset, numel
                _native.check(
                    lib.odc_convert(world.arena.handle, item, 1, native_dtype(src_dtype), native_dtype(dst_dtype), stream)
                )
            else:
                item = (_native.PublishItem * 1)()
                item[0].acc_offset = src_offset
                item[0].elems = numel
                peers = registry.peer_tensors[dst_key]
                for r in ranks:
                    item[0].out = peers[r].data_ptr()
                    _native.check(
                        lib.odc_publish(
                            world.arena.handle, r, item, 1, native_dtype(src_dtype), native_dtype(dst_dtype), 1.0, stream
                        )
                    )
            self._note_conversion(comm.cuda_stream)

    def _note_conversion(self, stream_handle: int) -> None:
        """A conversion was just launched on ``stream_handle``: gathers on other streams must
        not read its output before it is written. Conversions are rare (one per group and
        minibatch), so the event is recorded here, eagerly; a gather only looks at it when its
        own stream has not met this conversion yet."""
        if torch.cuda.is_current_stream_capturing():
            return  # inside a graph the capture's own stream order is all there is
        event = torch.cuda.Event()
        event.record(stream_from_handle(stream_handle))
        with self._lock:
            self._conversion = (stream_handle, event)
            self._met_conversion = {stream_handle}

    def _order_after_conversion(self, stream_handle: int) -> None:
        """Before a gather on ``stream_handle``: wait for the latest conversion if it ran on
        another stream and this stream has not waited for it yet."""
        if stream_handle in self._met_conversion:
            return
        with self._lock:
            if self._conversion is None or stream_handle in self._met_conversion:
                return
            if not torch.cuda.is_current_stream_capturing():
                stream_from_handle(stream_handle).wait_event(self._conversion[1])
                self._met_conversion = self._met_conversion | {stream_handle}
