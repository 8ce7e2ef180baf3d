"""CPU oracle for ODC's gather / scatter-accumulate path.

TEST INFRASTRUCTURE ONLY. Nothing in the product (``odc_amd/``) imports this module; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and
there only as the checker or the timed CPU baseline, never as the thing shipped.

Every function restates, with stock torch CPU ops, what the reference computes for W ranks; a
"world" here is simply a Python list indexed by rank. Citations are paths in the reference
repository (sail-sg/odc) or, where marked ``torch/``, in the PyTorch the reference patches.

How each function is pinned (tests/test_oracle.py):
  gather_cast               fp32->bf16 against the C restatement's integer round-to-nearest-even
                            on random values, ties and every exponent; widening casts are exact.
  fsdp1_publish / fsdp2_average   torch CPU div_ against exact rational arithmetic (fractions) on
                            samples and against the C restatement's binary32 division on random
                            values, denormals, zeros and infinities; the bf16 copy against the C
                            integer rounding.
  gather_into_tensor        closed-form ``i + 2r`` pattern of examples/all_gather.py:80-84,121-125;
                            brute-force Python loops on tiny inputs; sentinel bytes around dst.
  scatter_accumulate        closed forms (ones x M == M, powers of two, +0 + -0 == +0, Inf/NaN);
                            an independent scalar C restatement (oracle/odc_oracle.c) on random
                            and on all 2^16 bf16 bit patterns; split-size invariance; the
                            reduce-scatter equivalence of examples/reduce_scatter.py:96-105,163-172.
  BufferSplitter            table of hand-computed values.
  fsdp1_* / fsdp2_*         torch.chunk / F.pad / torch._chunk_cat / torch.split_with_sizes_copy
                            against index-by-index Python loops.
Bit-level parity of the fp32 add is not pinned by the reference itself (its only check is
rtol=atol=5e-3, examples/reduce_scatter.py:163-172); it is pinned by IEEE-754 semantics through
the checks above.
"""

from __future__ import annotations

import math
import os
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------
# gather
# --------------------------------------------------------------------------------------------
def gather_into_tensor(
    output: torch.Tensor, shards: Sequence[torch.Tensor], local_rank: int = 0
) -> torch.Tensor:
    """odc/primitives/gather.py:116-127 — ``output.view(W,-1)[src].copy_(peer[src])`` for
    ``src = (local_rank + k) % W``; the rotation only orders the copies."""
    W = len(shards)
    split = output.view(W, -1)
    for k in range(W):
        src = (local_rank + k) % W
        split[src].copy_(shards[src])
    return output


def gather(shards: Sequence[torch.Tensor]) -> torch.Tensor:
    """The same result as a fresh tensor: ``torch.cat`` of the W shards."""
    return torch.cat([s.reshape(-1) for s in shards])


def gather_cast(shards: Sequence[torch.Tensor], dtype: torch.dtype) -> torch.Tensor:
    """Gather in the shards' dtype, then convert the full parameter: odc/fsdp/fsdp1.py:199-223
    (``padded_unsharded_flat_param.copy_(…orig_dtype)``) and odc/fsdp/fsdp2.py:341-343
    (``_to_dtype_if_needed(all_gather_output, param_dtype)``). torch's conversion rounds to
    nearest even."""
    return gather(shards).to(dtype)


# --------------------------------------------------------------------------------------------
# buffer splitting (integer closed forms)
# --------------------------------------------------------------------------------------------
class BufferSplitter:
    """odc/primitives/utils.py:212-242."""

    round_data_size = 64

    def __init__(self, max_buffer_size: Optional[int] = None):
        if max_buffer_size is None:
            max_buffer_size = int(os.environ.get("ODC_MAX_BUFFER_SIZE", 64 * 1024 * 1024))
        self.max_buffer_size = max_buffer_size

    def get_global_buffer_size(self, shape) -> int:
        numel = math.prod(shape)
        if self.max_buffer_size <= 0:
            return numel
        return min(self.max_buffer_size, numel)

    def get_local_buffer_size(self, shape, world_size: int) -> int:
        numel = math.prod(shape)
        if self.max_buffer_size <= 0:
            size = numel
        else:
            if self.max_buffer_size % world_size != 0:
                raise AssertionError(
                    f"ODC_MAX_BUFFER_SIZE: {self.max_buffer_size} % world_size: {world_size} != 0"
                )
            size = min(self.max_buffer_size // world_size, numel)
        return (size + 63) // 64 * 64


# --------------------------------------------------------------------------------------------
# scatter-accumulate
# --------------------------------------------------------------------------------------------
def scatter_accumulate(
    accs: Sequence[torch.Tensor], grad: torch.Tensor, local_buf_size: Optional[int] = None
) -> None:
    """One client's ``ReductionService.scatter_accumulate`` as seen by the W owners.

    Client side (scatter_accumulate.py:649-669): for each sub-request ``start`` (step
    ``local_buf_size``) chunk r's slice ``grad[r*S + start : r*S + start + size]`` is staged on
    owner r. Owner side (scatter_accumulate.py:381-391): ``acc[start:start+size].add_(buf[:size])``
    with a running ``start``. ``accs[r]`` is owner r's accumulation (any of fp32/bf16/fp16), grad
    any of those; torch's mixed-dtype ``add_`` widens exactly, adds once in fp32 and rounds to the
    accumulation dtype.
    """
    W = len(accs)
    assert grad.dim() == 1 and grad.shape[0] % W == 0  # scatter_accumulate.py:589-592
    S = grad.shape[0] // W
    if local_buf_size is None or local_buf_size <= 0:
        local_buf_size = max(S, 1)
    chunks = grad.view(W, S)
    for r in range(W):
        acc = accs[r]
        assert acc.numel() == S
        start = 0
        while start < S:
            size = min(local_buf_size, S - start)
            buf = chunks[r, start : start + size].clone()  # the staging copy
            acc[start : start + size].add_(buf[:size])
            start += size


def clear_accumulations(accs: Sequence[torch.Tensor]) -> None:
    """scatter_accumulate.py:585-587."""
    for acc in accs:
        acc.fill_(0)


# --------------------------------------------------------------------------------------------
# FSDP1 flat-parameter layout
# --------------------------------------------------------------------------------------------
def fsdp1_get_shard(flat: torch.Tensor, rank: int, world_size: int) -> torch.Tensor:
    """torch/distributed/fsdp/_flat_param.py:1091-1142 as used by odc/fsdp/fsdp1.py:239-247:
    ``flat.chunk(W)[rank]`` right-padded with zeros to ``chunk(W)[0].numel()``; a rank beyond the
    last chunk holds only zeros."""
    chunks = torch.flatten(flat).chunk(world_size)
    if rank < len(chunks):
        chunk = chunks[rank].clone()
    else:
        chunk = chunks[0].new_empty(0)
    pad = chunks[0].numel() - chunk.numel()
    return F.pad(chunk, [0, pad]) if pad > 0 else chunk


def fsdp1_pad_grad(unsharded_grad: torch.Tensor, world_size: int) -> torch.Tensor:
    """odc/fsdp/fsdp1.py:25-38: right-pad the flat gradient with zeros to W * chunk0."""
    chunks = list(unsharded_grad.chunk(world_size))
    numel_to_pad = world_size * chunks[0].numel() - unsharded_grad.numel()
    return F.pad(unsharded_grad, [0, numel_to_pad]) if numel_to_pad > 0 else unsharded_grad


# --------------------------------------------------------------------------------------------
# FSDP2 parameter-group layout (dim-0 sharding)
# --------------------------------------------------------------------------------------------
def fsdp2_padded_shard_numel(shape: Sequence[int], world_size: int) -> int:
    """torch/distributed/fsdp/_fully_shard/_fsdp_common.py:109-111: dim 0 rounded up to a
    multiple of W, divided by W, times the trailing dims."""
    rest = math.prod(shape[1:])
    return math.ceil(shape[0] / world_size) * rest


def fsdp2_pack_shards(params: Sequence[torch.Tensor], world_size: int) -> List[torch.Tensor]:
    """odc/fsdp/fsdp2.py:146-196: rank r's group buffer is the concatenation over params of its
    zero-padded dim-0 chunk (torch/distributed/fsdp/_fully_shard/_fsdp_param.py
    ``_init_sharded_param``)."""
    out = []
    for r in range(world_size):
        pieces = []
        for p in params:
            n = fsdp2_padded_shard_numel(p.shape, world_size)
            chunks = torch.chunk(p, world_size, dim=0)
            piece = p.new_zeros(n)
            if r < len(chunks):
                piece[: chunks[r].numel()].copy_(chunks[r].reshape(-1))
            pieces.append(piece)
        out.append(torch.cat(pieces) if pieces else torch.empty(0))
    return out


def fsdp2_copy_out(
    gathered: torch.Tensor, shapes: Sequence[Sequence[int]], world_size: int
) -> List[torch.Tensor]:
    """odc/fsdp/fsdp2.py:378-401: split the ``[W, sum n_p]`` gathered buffer back into one padded
    unsharded tensor per param with ``split_with_sizes_copy(dim=1)``; param p then reads its
    first ``shape[0]`` rows."""
    sizes = [fsdp2_padded_shard_numel(s, world_size) for s in shapes]
    outs = [gathered.new_empty(world_size, n) for n in sizes]
    torch.split_with_sizes_copy(gathered.view(world_size, -1), sizes, dim=1, out=outs)
    result = []
    for o, s in zip(outs, shapes):
        rows = math.ceil(s[0] / world_size) * world_size
        result.append(o.view(rows, *s[1:])[: s[0]])
    return result


def fsdp2_copy_in(
    grads: Sequence[torch.Tensor], world_size: int, reduce_dtype: torch.dtype
) -> torch.Tensor:
    """odc/fsdp/fsdp2.py:671-682 -> torch/distributed/fsdp/_fully_shard/_fsdp_collectives.py:666-674:
    ``torch._chunk_cat`` pads dim 0 of every gradient to a multiple of W, casts to the reduce
    dtype and lays the result out as ``[W, sum n_p]``."""
    total = sum(fsdp2_padded_shard_numel(g.shape, world_size) for g in grads) * world_size
    out = torch.empty(total, dtype=reduce_dtype)
    torch._chunk_cat(list(grads), dim=0, num_chunks=world_size, out=out.view(world_size, -1))
    return out


def fsdp2_grad_views(
    acc: torch.Tensor, shapes: Sequence[Sequence[int]], world_size: int, rank: int
) -> List[torch.Tensor]:
    """odc/fsdp/fsdp2.py:897-932: rank ``rank``'s sharded gradients as ``as_strided`` views of
    its accumulation buffer, offset advancing by the padded shard numel."""
    views = []
    offset = 0
    for s in shapes:
        chunk_rows = math.ceil(s[0] / world_size)
        rows = max(0, min(chunk_rows, s[0] - rank * chunk_rows))
        size = (rows, *s[1:])
        stride = torch.empty(max(rows, 1), *s[1:]).stride()  # contiguous strides of the shard
        views.append(
            torch.as_strided(acc, size=size, stride=stride, storage_offset=acc.storage_offset() + offset)
        )
        offset += fsdp2_padded_shard_numel(s, world_size)
    return views


# --------------------------------------------------------------------------------------------
# minibatch hooks
# --------------------------------------------------------------------------------------------
def fsdp1_publish(acc: torch.Tensor, postdivide_factor: float, param_dtype: torch.dtype):
    """odc/fsdp/fsdp1.py:324-335: ``_div_if_needed(acc, factor)`` in place
    (torch/distributed/fsdp/_runtime_utils.py ``_div_if_needed``: divide when factor > 1), then
    ``acc.to(param_dtype)`` becomes ``flat_param.grad``."""
    if postdivide_factor > 1:
        acc.div_(postdivide_factor)
    return acc.to(param_dtype)


def fsdp2_average(acc: torch.Tensor, world_size: int) -> torch.Tensor:
    """odc/fsdp/fsdp2.py:846-847: ``reduce_output /= world_size`` in place for ReduceOp.AVG."""
    acc /= world_size
    return acc
