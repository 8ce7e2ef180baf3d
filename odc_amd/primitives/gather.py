"""On-demand gather: W sharded buffers -> one full flat buffer, one fused HIP launch.

Mirror of ``odc/primitives/gather.py`` (``GatherService.gather_into_tensor``, :76-127,176). The
reference issues W peer ``copy_``s on a side stream; here the same result comes from
``odc_gather`` (include/odc_hip.h), whose work list covers all W shards of all tensors of the
call. The inter-node NVSHMEM branch of the reference (:129-175) has no counterpart on one GPU.
"""

from __future__ import annotations

import ctypes
import logging
from typing import Sequence

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
)

logger = logging.getLogger(__name__)


class GatherService:
    def __init__(self):
        self.buffer_splitter = BufferSplitter()

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
        get_world()  # raises when there is no arena (no GPU, or init_nvshmem not called)
        registry = SymmBufferRegistry.get_instance()
        pairs = [(o, i) for o, i in zip(output_tensors, input_tensors) if i.numel() or o.numel()]
        if not pairs:
            return
        for _, inp in pairs:
            assert inp.is_cuda and inp.is_contiguous(), "shards are contiguous GPU tensors"
            assert inp.dtype == pairs[0][1].dtype, "one launch takes one dtype pair"
        self._gather(
            [o for o, _ in pairs],
            [registry.symmetric_offset_of(i) for _, i in pairs],
            [i.numel() for _, i in pairs],
            pairs[0][1].dtype,
            pg,
        )

    def _gather(self, outs, src_offsets, shard_numels, src_dtype, pg) -> None:
        """One launch (per 64 items): ``outs[k].view(W, -1)[r]`` = the ``shard_numels[k]`` elements
        of ``src_dtype`` at symmetric byte offset ``src_offsets[k]`` of rank r."""
        world = get_world()
        W = group_size(pg)
        assert W == world.world_size, f"group size {W} != arena world size {world.world_size}"
        dst_dtype = outs[0].dtype
        cast = src_dtype != dst_dtype
        es = src_dtype.itemsize
        items = ((_native.GatherCastItem if cast else _native.GatherItem) * len(outs))()
        for item, out, offset, n in zip(items, outs, src_offsets, shard_numels):
            assert out.is_cuda, "gather runs on the GPU only"
            assert out.dtype == dst_dtype, "one launch takes one dtype pair"
            assert out.is_contiguous()
            assert out.numel() == W * n, f"output numel {out.numel()} != {W} * shard numel {n}"
            item.dst = out.data_ptr()
            item.src_offset = offset
            if cast:
                item.shard_elems = n
            else:
                item.shard_bytes = n * es

        lib = _native.load()
        with comm_stream_section(f"odc.gather[{len(items)}]") as comm:
            stream = ctypes.c_void_p(comm.cuda_stream)
            if cast:
                # shards kept in one dtype (fp32 master copies), full parameter wanted in another
                # (bf16): converted on the way instead of gathered and then cast
                # (odc/fsdp/fsdp1.py:199-223, odc/fsdp/fsdp2.py:341-343)
                status = lib.odc_gather_cast(
                    world.arena.handle, items, len(items), native_dtype(src_dtype),
                    native_dtype(dst_dtype), get_rank(), stream,
                )
            else:
                status = lib.odc_gather(world.arena.handle, items, len(items), get_rank(), stream)
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
        es = input_tensor.element_size()
        base = SymmBufferRegistry.get_instance().symmetric_offset_of(input_tensor)
        outs, offsets, numels = [], [], []
        for out, off, n in zip(output_tensors, slice_offsets, slice_numels):
            assert 0 <= off and off + n <= input_tensor.numel(), "slice leaves the buffer"
            if n or out.numel():
                outs.append(out)
                offsets.append(base + off * es)
                numels.append(n)
        if outs:
            self._gather(outs, offsets, numels, input_tensor.dtype, pg)
