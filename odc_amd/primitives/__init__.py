"""gather / scatter-accumulate primitives and the symmetric-memory registry.

The reference's package init (``odc/primitives/__init__.py``) imports its Triton/NVSHMEM
externs and the ``tensor_ipc`` extension and fails if the latter is not built; here the one
native dependency is ``libodc_hip.so``, loaded (and required) on import.
"""

from odc_amd import _native

_native.load()  # raises ImportError when the HIP library has not been built

from odc_amd.primitives.gather import GatherService  # noqa: E402
from odc_amd.primitives.scatter_accumulate import ReductionService  # noqa: E402
from odc_amd.primitives.tensor_ipc import get_ipc_handle, reconstruct_tensor  # noqa: E402
from odc_amd.primitives.utils import (  # noqa: E402
    BufferSplitter,
    SymmBufferRegistry,
    VirtualGroup,
    finalize_distributed,
    get_comm_stream,
    get_local_world_size,
    get_rank,
    get_world_size,
    init_nvshmem,
    set_rank,
    virtual_rank,
)

__all__ = [
    "GatherService",
    "ReductionService",
    "SymmBufferRegistry",
    "BufferSplitter",
    "VirtualGroup",
    "init_nvshmem",
    "finalize_distributed",
    "get_comm_stream",
    "get_local_world_size",
    "get_rank",
    "get_world_size",
    "set_rank",
    "virtual_rank",
    "get_ipc_handle",
    "reconstruct_tensor",
]
