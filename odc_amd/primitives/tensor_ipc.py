"""In-process counterpart of the reference's ``tensor_ipc`` extension
(``csrc/tensor_ipc/tensor_ipc.cu:24-57``, bound in ``csrc/tensor_ipc/binding.cpp:8-11``).

There a handle is a CUDA IPC memory handle of the allocation plus the tensor's offset inside
it (72 bytes), and ``reconstruct_tensor`` opens it in the watcher process. Here every rank's
memory lives in one arena of one process, so a handle is the arena's identity plus (rank,
offset): ``odc_arena_locate`` on the way out, ``odc_arena_ptr`` on the way back. The handle
keeps the 72-byte size so that code which stores or ships it unchanged keeps working; opening
it in another process is not possible (and not needed: owner and caller share the process).
"""

from __future__ import annotations

import struct
from typing import Sequence

import torch

from odc_amd.primitives.utils import get_world

_MAGIC = b"ODCHIP01"
_LAYOUT = struct.Struct("<8sQQIQ")  # magic, arena base, rank stride, rank, byte offset
HANDLE_BYTES = 72


def get_ipc_handle(tensor: torch.Tensor) -> bytes:
    """Handle of a tensor that lives in the symmetric arena (any rank's view, any inner offset)."""
    arena = get_world().arena
    rank, alloc_offset, inner = arena.locate(tensor.data_ptr())
    info = arena.info()
    packed = _LAYOUT.pack(_MAGIC, info.base, info.rank_stride, rank, alloc_offset + inner)
    return packed + bytes(HANDLE_BYTES - len(packed))


def reconstruct_tensor(handle: bytes, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
    """A non-owning tensor of ``shape`` and ``dtype`` at the handle's address."""
    if len(handle) != HANDLE_BYTES:
        raise ValueError(f"handle must be {HANDLE_BYTES} bytes, got {len(handle)}")
    magic, base, stride, rank, offset = _LAYOUT.unpack_from(handle)
    arena = get_world().arena
    info = arena.info()
    if magic != _MAGIC or base != info.base or stride != info.rank_stride:
        raise ValueError("handle does not belong to this process's symmetric arena")
    return arena.view(rank, offset, tuple(shape), dtype)
