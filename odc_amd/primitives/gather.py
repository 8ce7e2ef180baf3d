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

import torch
from torch import Tensor

from odc_amd import _native
from odc_amd.primitives.utils import (
    BufferSplitter,
    SymmBufferRegistry,
    get_comm_stream,
    get_rank,
    get_world,
    group_size,
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
        """Multi-tensor form: every (output, input) pair of the lists in ONE launch (per 32
        pairs). Equivalent to calling ``gather_into_tensor`` pair by pair."""
        assert len(output_tensors) == len(input_tensors)
        world = get_world()
        W = group_size(pg)
        assert W == world.world_size, f"group size {W} != arena world size {world.world_size}"
        registry = SymmBufferRegistry.get_instance()
        pairs = [(o, i) for o, i in zip(output_tensors, input_tensors) if i.numel() or o.numel()]
        items = (_native.GatherItem * max(len(pairs), 1))()
        for i, (out, inp) in enumerate(pairs):
            assert out.is_cuda and inp.is_cuda, "gather runs on the GPU only"
            assert out.dtype == inp.dtype, f"{out.dtype=} != {inp.dtype=}"
            assert out.is_contiguous() and inp.is_contiguous()
            assert (
                out.numel() == W * inp.numel()
            ), f"output numel {out.numel()} != {W} * shard numel {inp.numel()}"
            items[i].dst = out.data_ptr()
            items[i].src_offset = registry.symmetric_offset_of(inp)
            items[i].shard_bytes = inp.numel() * inp.element_size()

        comm = get_comm_stream()
        comm.wait_stream(torch.cuda.current_stream())
        _native.check(
            _native.load().odc_gather(
                world.arena.handle, items, len(pairs), get_rank(), ctypes.c_void_p(comm.cuda_stream)
            )
        )
        torch.cuda.current_stream().wait_stream(comm)
