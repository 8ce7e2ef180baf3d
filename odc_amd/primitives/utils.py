"""Symmetric memory for W virtual ranks on one MI355X.

Host-side mirror of ``odc/primitives/utils.py``: the same names (``init_nvshmem``,
``finalize_distributed``, ``SymmBufferRegistry``, ``BufferSplitter``, ``get_comm_stream``,
``get_local_world_size``) with the NVSHMEM symmetric heap replaced by the arena of
``libodc_hip.so``: one ``hipMalloc`` cut into W rank regions, where one byte offset names the
same buffer in every region. A *virtual rank* is one of those regions; the process plays any of
them (``set_rank`` / ``virtual_rank``) the way one process per GPU plays its rank in the
reference.
"""

from __future__ import annotations

import contextlib
import ctypes
import logging
import math
import os
import threading
from functools import reduce
from typing import List, Optional

import torch

from odc_amd import _native

logger = logging.getLogger(__name__)

_SIZE_SUFFIX = {"K": 2**10, "M": 2**20, "G": 2**30, "T": 2**40}


def parse_size(text) -> int:
    """'30G', '5000000000', '512M' -> bytes (the forms NVSHMEM_SYMMETRIC_SIZE takes,
    launch.sh:135, README.md:53-57)."""
    if isinstance(text, int):
        return text
    s = str(text).strip().upper().rstrip("B")
    if s and s[-1] in _SIZE_SUFFIX:
        return int(float(s[:-1]) * _SIZE_SUFFIX[s[-1]])
    return int(s)


_TORCH_TO_NATIVE = {
    torch.bfloat16: _native.DTYPE_BF16,
    torch.float16: _native.DTYPE_F16,
    torch.float32: _native.DTYPE_F32,
}


def native_dtype(dtype: torch.dtype) -> int:
    try:
        return _TORCH_TO_NATIVE[dtype]
    except KeyError:
        raise TypeError(f"scatter-accumulate supports bf16/fp16/fp32, not {dtype}") from None


class VirtualGroup:
    """Stands in for a ``torch.distributed.ProcessGroup`` wherever the reference takes ``pg``:
    W virtual ranks living in one HBM. Only ``size()`` and ``rank()`` are ever asked of it."""

    def __init__(self, world_size: int):
        self._world_size = int(world_size)

    def size(self) -> int:
        return self._world_size

    def rank(self) -> int:
        return get_rank()

    def __repr__(self):
        return f"VirtualGroup(world_size={self._world_size})"


def group_size(pg) -> int:
    """``torch.distributed.get_world_size(pg)`` for real and virtual groups; None = the world."""
    if pg is None:
        return get_world().world_size
    return pg.size()


class _ArenaMemory:
    """Exposes the arena to torch through ``__cuda_array_interface__`` (zero copy, non-owning)."""

    def __init__(self, ptr: int, nbytes: int):
        self.__cuda_array_interface__ = {
            "shape": (nbytes,),
            "typestr": "|u1",
            "data": (ptr, False),
            "version": 2,
            "strides": None,
        }


class SymmetricArena:
    """Python handle of one ``odc_arena`` (include/odc_hip.h)."""

    def __init__(self, world_size: int, bytes_per_rank: int, backing: bool = True):
        self._lib = _native.load()
        self._handle = ctypes.c_void_p()
        flags = _native.ODC_ARENA_DEVICE if backing else _native.ODC_ARENA_NO_BACKING
        _native.check(
            self._lib.odc_arena_create(
                int(world_size), int(bytes_per_rank), flags, ctypes.byref(self._handle)
            )
        )
        info = self.info()
        self.world_size = info.world_size
        self.bytes_per_rank = info.bytes_per_rank
        self.rank_stride = info.rank_stride
        self.base = info.base
        self.device = info.device
        self._bytes = None
        if backing:
            mem = _ArenaMemory(self.base, self.rank_stride * self.world_size)
            self._bytes = torch.as_tensor(mem, device=torch.device("cuda", self.device))
            assert self._bytes.data_ptr() == self.base, "torch did not alias the arena"

    @property
    def handle(self):
        if self._handle is None or not self._handle.value:
            raise RuntimeError("the symmetric arena has been finalized")
        return self._handle

    def info(self) -> _native.ArenaInfo:
        info = _native.ArenaInfo()
        _native.check(self._lib.odc_arena_get_info(self.handle, ctypes.byref(info)))
        return info

    def alloc(self, nbytes: int) -> int:
        off = ctypes.c_uint64()
        _native.check(self._lib.odc_arena_alloc(self.handle, int(nbytes), ctypes.byref(off)))
        return off.value

    def free(self, offset: int) -> None:
        _native.check(self._lib.odc_arena_free(self.handle, int(offset)))

    def reset(self) -> None:
        _native.check(self._lib.odc_arena_reset(self.handle))

    def ptr(self, rank: int, offset: int) -> int:
        p = self._lib.odc_arena_ptr(self.handle, int(rank), int(offset))
        if not p:
            raise _native.OdcNativeError(
                _native.ODC_ERR_INVALID, self._lib.odc_last_error().decode()
            )
        return p

    def locate(self, ptr: int):
        """device address -> (rank, allocation offset, distance into the allocation)."""
        rank, off, inner = ctypes.c_uint32(), ctypes.c_uint64(), ctypes.c_uint64()
        _native.check(
            self._lib.odc_arena_locate(
                self.handle, ctypes.c_void_p(ptr), ctypes.byref(rank), ctypes.byref(off),
                ctypes.byref(inner),
            )
        )
        return rank.value, off.value, inner.value

    def view(self, rank: int, offset: int, shape, dtype: torch.dtype) -> torch.Tensor:
        """Non-owning tensor over rank ``rank``'s copy of the buffer at ``offset``."""
        if self._bytes is None:
            raise RuntimeError("a bookkeeping-only arena has no memory to view")
        numel = reduce(lambda x, y: x * y, shape, 1)
        nbytes = numel * dtype.itemsize
        if not 0 <= rank < self.world_size or offset + nbytes > self.bytes_per_rank:
            raise ValueError(f"view of rank {rank} [{offset}, +{nbytes}) leaves the rank region")
        if nbytes == 0:
            return torch.empty(tuple(shape), dtype=dtype, device=self._bytes.device)
        # a tensor of its own (storage offset 0), so that callers may as_strided into it with
        # absolute offsets the way odc/fsdp/fsdp2.py:902-907 does
        mem = _ArenaMemory(self.base + rank * self.rank_stride + offset, nbytes)
        flat = torch.as_tensor(mem, device=self._bytes.device)
        return flat.view(dtype).view(tuple(shape))

    def destroy(self) -> None:
        if self._handle is not None and self._handle.value:
            self._bytes = None
            handle, self._handle = self._handle, None
            _native.check(self._lib.odc_arena_destroy(handle))


_world_serial = 0


class _VirtualWorld:
    def __init__(self, arena: SymmetricArena):
        global _world_serial
        _world_serial += 1
        self.serial = _world_serial  # tells one arena from the next in caches that outlive it
        self.arena = arena
        self.world_size = arena.world_size
        self.rank = 0
        self.group = VirtualGroup(self.world_size)


_world: Optional[_VirtualWorld] = None


def get_world() -> _VirtualWorld:
    if _world is None:
        raise RuntimeError("init_nvshmem() has not been called: there is no symmetric arena")
    return _world


def is_initialized() -> bool:
    return _world is not None


def init_nvshmem(world_size: Optional[int] = None, symmetric_size=None):
    """Create the symmetric arena (the name is the reference's, ``utils.py:18-49``, where it boots
    NVSHMEM over the global process group).

    ``world_size``: number of virtual ranks W; default ``$ODC_VIRTUAL_WORLD_SIZE``, else
    ``get_local_world_size()``. ``symmetric_size``: bytes per rank; default
    ``$ODC_SYMMETRIC_SIZE``, else ``$NVSHMEM_SYMMETRIC_SIZE`` (the reference's knob,
    ``launch.sh:135``), else 1 GiB. Returns the world's ``VirtualGroup``.
    """
    global _world
    if _world is not None:
        raise RuntimeError("init_nvshmem() called twice without finalize_distributed()")
    if world_size is None:
        env = os.environ.get("ODC_VIRTUAL_WORLD_SIZE")
        world_size = int(env) if env else get_local_world_size()
    if symmetric_size is None:
        symmetric_size = os.environ.get(
            "ODC_SYMMETRIC_SIZE", os.environ.get("NVSHMEM_SYMMETRIC_SIZE", "1G")
        )
    nbytes = parse_size(symmetric_size)
    if not torch.cuda.is_available():
        raise RuntimeError("init_nvshmem() needs a GPU: the symmetric arena lives in HBM")
    _world = _VirtualWorld(SymmetricArena(world_size, nbytes))
    logger.info(f"symmetric arena: {world_size} ranks x {nbytes} bytes")
    return _world.group


def finalize_distributed():
    """Release the arena (``utils.py:84-85``). Tensors handed out by the registry dangle after
    this, exactly as NVSHMEM tensors do after ``nvshmem.core.finalize``."""
    global _world, stream
    if _world is not None:
        if hasattr(SymmBufferRegistry, "_instance"):
            SymmBufferRegistry._instance._forget()
        _world.arena.destroy()
        _world = None
    _bare_allocations.clear()
    with _launch_lock:
        _launch_streams.clear()  # handles of a world that is gone are not waited for
    stream = None


# symmetric allocations made through the reference's bare helpers: local data_ptr -> (offset, shape, dtype)
_bare_allocations = {}


def nvshmem_create_tensor(shape, dtype) -> torch.Tensor:
    """A symmetric tensor outside the registry (``utils.py:53-57``): the calling rank's view of
    a fresh arena allocation that exists, at the same offset, in every rank region."""
    world = get_world()
    shape = tuple(shape) if not isinstance(shape, int) else (shape,)
    offset = world.arena.alloc(max(1, math.prod(shape)) * dtype.itemsize)
    tensor = world.arena.view(get_rank(), offset, shape, dtype)
    _bare_allocations[tensor.data_ptr()] = (offset, shape, dtype)
    return tensor


def get_same_node_tensors(tensor, rank, local_world_size) -> List[torch.Tensor]:
    """The views of ``tensor``'s symmetric allocation on every rank of ``rank``'s node
    (``utils.py:60-75``); the entry for ``rank`` is ``tensor`` itself. ``tensor`` is any
    symmetric tensor of any rank: made by ``nvshmem_create_tensor`` or by the registry."""
    world = get_world()
    _owner, offset, inner = world.arena.locate(tensor.data_ptr())
    first = rank - rank % local_world_size
    return [
        tensor if peer == rank else world.arena.view(peer, offset + inner, tuple(tensor.shape), tensor.dtype)
        for peer in range(first, first + local_world_size)
    ]


def nvshmem_free_tensor_sync(tensor) -> None:
    """Free a tensor made by ``nvshmem_create_tensor`` (``utils.py:78-81``), after the device has
    finished with it. The tensor and its peers dangle afterwards."""
    entry = _bare_allocations.pop(tensor.data_ptr(), None)
    if entry is None:
        raise ValueError("tensor was not made by nvshmem_create_tensor (or was freed already)")
    torch.cuda.synchronize()
    get_world().arena.free(entry[0])


def get_local_world_pg(pg):
    """The group of the calling rank's node (``utils.py:178-192``). All W virtual ranks share
    one GPU, hence one node: the group itself."""
    assert group_size(pg) == get_world().world_size, "the group must span the virtual world"
    return pg


def get_rank() -> int:
    """The virtual rank this process currently plays (``torch.distributed.get_rank()`` there)."""
    return get_world().rank


def get_world_size() -> int:
    return get_world().world_size


def set_rank(rank: int) -> None:
    world = get_world()
    if not 0 <= rank < world.world_size:
        raise ValueError(f"rank {rank} outside [0, {world.world_size})")
    world.rank = int(rank)


@contextlib.contextmanager
def virtual_rank(rank: int):
    """``with virtual_rank(r):`` — act as rank r, then return to the previous rank."""
    prev = get_rank()
    set_rank(rank)
    try:
        yield
    finally:
        set_rank(prev)


class SymmBufferRegistry:
    """name -> symmetric buffer, ``utils.py:88-172``.

    ``local_tensor[key]`` is the current rank's view at the time of the lookup;
    ``peer_tensors[key]`` are all W views. Both alias arena memory and own nothing.
    """

    def __init__(self, arena=None, rank_fn=None):
        # arena/rank_fn default to the process-wide virtual world; passing them gives a
        # registry of its own (used to exercise the bookkeeping without a GPU)
        self._arena = arena
        self._rank_fn = rank_fn
        self.offsets = {}  # key -> (offset, shape, dtype)
        self.local_tensor_to_keys = {}  # data_ptr of any rank's view -> key
        self.updated = set()  # (key, rank)
        self.peer_tensors = {}
        self.allocations = []

    @property
    def arena(self):
        return self._arena if self._arena is not None else get_world().arena

    @classmethod
    def get_instance(cls):
        if not hasattr(cls, "_instance"):
            cls._instance = SymmBufferRegistry()
        return cls._instance

    @property
    def local_tensor(self):
        """key -> the current rank's tensor (a fresh dict; the reference's attribute of the
        same name, read by ``fsdp2.get_symm_buffer_memory_breakdown``)."""
        rank = self._rank()
        return {k: peers[rank] for k, peers in self.peer_tensors.items()}

    def _rank(self) -> int:
        return self._rank_fn() if self._rank_fn is not None else get_rank()

    # we'll mark all symm buffers dirty; the next update_symm_buffer copies again
    def flush(self):
        self.updated.clear()

    def update_symm_buffer(self, buffer_key, values):
        values = values.contiguous()
        if buffer_key not in self.peer_tensors:
            self.allocate_symm_buffer(buffer_key, values.shape, values.dtype)
        rank = self._rank()
        local = self.peer_tensors[buffer_key][rank]
        if (buffer_key, rank) not in self.updated:
            self.updated.add((buffer_key, rank))
            local.copy_(values)
            # the reference barriers here so that peers see the shard; with one process the
            # copy is ordered before later work on the same stream, and gather's stream join
            # (comm_stream.wait_stream(current)) orders it before any read.
        return local

    @classmethod
    def set_nvshmem_flag(cls, tensor):
        tensor._odc_is_nvshmem = True

    @classmethod
    def is_nvshmem_tensor(cls, tensor):
        return hasattr(tensor, "_odc_is_nvshmem") and tensor._odc_is_nvshmem

    def allocate_symm_buffer(self, key, shape, dtype):
        assert key not in self.peer_tensors
        arena = self.arena
        shape = tuple(shape)
        numel = reduce(lambda x, y: x * y, shape, 1)
        offset = arena.alloc(numel * dtype.itemsize)
        peers = [arena.view(r, offset, shape, dtype) for r in range(arena.world_size)]
        for t in peers:
            self.set_nvshmem_flag(t)
            self.local_tensor_to_keys[t.data_ptr()] = key
        self.allocations.append(peers[0])
        self.offsets[key] = (offset, shape, dtype)
        self.peer_tensors[key] = peers
        local = peers[self._rank()]
        logger.info(
            f"Rank {self._rank()} create tensor {key} with shape {shape} and dtype {dtype} "
            f"and ptr {local.data_ptr()}"
        )
        return local

    def has_key(self, key):
        return key in self.peer_tensors

    def get_or_create_symm_buffer(self, key, shape, dtype):
        if self.has_key(key):
            return self.peer_tensors[key][self._rank()]
        return self.allocate_symm_buffer(key, shape, dtype)

    def get_symm_buffer(self, key):
        if self.has_key(key):
            return self.peer_tensors[key][self._rank()]
        raise ValueError(f"Symm buffer {key} not found")

    def get_peer_tensors(self, local_tensor) -> List[torch.Tensor]:
        buffer_key = self.local_tensor_to_keys[local_tensor.data_ptr()]
        return self.peer_tensors[buffer_key]

    def get_offset(self, key) -> int:
        """Symmetric byte offset of a registered buffer (what the kernels take)."""
        return self.offsets[key][0]

    def symmetric_offset_of(self, tensor: torch.Tensor) -> int:
        """Symmetric byte offset of ``tensor``, which must be (a contiguous view into) a
        registered buffer of any rank. Exact buffer starts resolve through the data_ptr map
        (``utils.py:158-161``); inner views through ``odc_arena_locate``."""
        key = self.local_tensor_to_keys.get(tensor.data_ptr())
        if key is not None:
            return self.offsets[key][0]
        if not tensor.is_cuda:
            raise ValueError("tensor is not in the symmetric arena")
        try:
            _rank, off, inner = self.arena.locate(tensor.data_ptr())
        except _native.OdcNativeError as e:
            raise ValueError(f"tensor is not in the symmetric arena: {e.message}") from None
        return off + inner

    def _forget(self):
        self.offsets.clear()
        self.local_tensor_to_keys.clear()
        self.updated.clear()
        self.peer_tensors.clear()
        self.allocations.clear()

    def finalize(self):
        arena = self.arena if (self._arena is not None or is_initialized()) else None
        if arena is not None:
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            for offset, _shape, _dtype in self.offsets.values():
                arena.free(offset)
        self._forget()

    def memory_allocated(self):
        return sum(t.nbytes for t in self.allocations)


def get_local_world_size():
    """Ranks per node (``utils.py:195-199``); here it is also the default number of virtual ranks."""
    if _world is not None:
        return _world.world_size
    if "RAY_LOCAL_WORLD_SIZE" in os.environ:
        return int(os.environ["RAY_LOCAL_WORLD_SIZE"])
    else:
        return int(os.environ["LOCAL_WORLD_SIZE"])


stream = None
_stream_lock = threading.Lock()


def get_comm_stream():
    """One side stream for all primitive launches (``utils.py:205-209``), default priority.
    Callers may come from several host threads (autograd's device thread in backward)."""
    global stream
    if stream is None:
        with _stream_lock:
            if stream is None:
                stream = torch.cuda.Stream()
    return stream


_launch_streams = {}  # stream handle -> torch stream with launches since the last wait (None: not wrapped yet)
_launch_lock = threading.Lock()  # launches come from several host threads (autograd's device thread)


def stream_from_handle(handle: int):
    """A torch stream object for a raw stream handle of the arena's device."""
    device = get_world().arena.device
    if handle == 0:  # the default stream: ExternalStream does not wrap a null handle
        return torch.cuda.default_stream(device)
    return torch.cuda.ExternalStream(handle, device=device)


class StreamOrder:
    """Orders launches that touch the same buffer from different streams.

    In the reference every add into a rank's accumulation goes through that rank's one watcher
    (``scatter_accumulate.py:291-310,386-392``), so clients on different streams never race on
    it. Here a launch is a plain read-modify-write on the caller's stream; this class remembers,
    per key, the stream of the last launch that wrote it, and when the next launch for that key
    comes on another stream it makes the new stream wait for an event recorded on the previous
    one. Nothing is recorded while launches stay on one stream (the steady state: one comparison
    per call). Not thread safe on its own: the owner calls it under its lock.

    Launches recorded into a HIP graph are not tracked: a graph runs on whatever stream it is
    replayed on, which the host cannot know at capture time; ordering a replay against eager
    launches on other streams is the caller's business, as it is for any graph."""

    __slots__ = ("_base", "_last")

    def __init__(self):
        self._base = None  # the stream every key without an entry in _last was last written on
        self._last = {}  # key -> stream handle, for the keys that differ from _base

    def forget(self):
        self._base = None
        self._last.clear()

    def before_launch(self, keys, handle: int, all_keys: bool = False, total: int = 0) -> None:
        """Call before launching work that writes ``keys`` on stream ``handle``. ``all_keys``:
        the launch writes every key there is; ``total``: how many keys there are (lets the
        per-key table collapse once all of them have moved to one stream)."""
        if not self._last:
            if self._base == handle:
                return
            if self._base is None:
                self._base = handle
                return
        previous = set()
        if all_keys:
            previous.update(self._last.values())
            previous.add(self._base)
            self._last.clear()
            self._base = handle
        else:
            last, base = self._last, self._base
            for key in keys:
                previous.add(last.get(key, base))
                if handle == base:
                    last.pop(key, None)
                else:
                    last[key] = handle
            if total and len(last) >= total and all(h == handle for h in last.values()):
                last.clear()
                self._base = handle
        previous.discard(handle)
        previous.discard(None)
        if previous:
            current = stream_from_handle(handle)
            for prev in previous:
                join_streams(current, prev)


def join_streams(current, previous_handle: int) -> None:
    """Make ``current`` wait for everything queued so far on the stream ``previous_handle``."""
    event = torch.cuda.Event()
    try:
        event.record(stream_from_handle(previous_handle))
    except RuntimeError:
        # the stream no longer exists (a user stream destroyed since its launch); what it had
        # queued may still be running, and only the device as a whole can be waited for
        torch.cuda.synchronize(get_world().arena.device)
        return
    current.wait_event(event)

# The two environment switches are read on every launch, so that they can be flipped at run time;
# os.environ.get costs a microsecond per lookup (key encoding), the mapping underneath it does not.
_ENVIRON_DATA = getattr(os.environ, "_data", None)
_ENCODE_KEY = getattr(os.environ, "encodekey", None)


def _fast_env_reader(name: str):
    if isinstance(_ENVIRON_DATA, dict) and _ENCODE_KEY is not None:
        try:
            key, decode = _ENCODE_KEY(name), os.environ.decodevalue
            return lambda: decode(_ENVIRON_DATA[key]) if key in _ENVIRON_DATA else None
        except Exception:  # an os.environ without these internals: the documented way
            pass
    return lambda: os.environ.get(name)


_read_policy = _fast_env_reader("ODC_COMM_STREAM")
_read_trace = _fast_env_reader("ODC_TRACE")


def launch_stream_policy() -> str:
    """``ODC_COMM_STREAM``: "caller" (default) launches on the caller's current stream;
    "dedicated" hops to the one comm stream and joins it on both sides, as the reference does."""
    policy = _read_policy()
    if policy is None or policy == "caller":
        return "caller"
    if policy != "dedicated":
        raise ValueError(f"ODC_COMM_STREAM must be 'caller' or 'dedicated', not {policy!r}")
    return policy


def _tracing() -> bool:
    return _read_trace() == "1"


_current_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
if _current_raw_stream is None:  # a torch without the raw accessor: ask for the stream object

    def _current_raw_stream(device: int) -> int:
        return torch.cuda.current_stream(device).cuda_stream


class comm_stream_section:
    """``with comm_stream_section(label) as section:`` — ``section.cuda_stream`` is the handle of
    the stream the body's launches go to.
    With ``ODC_TRACE=1`` the section is a marker range named ``label`` (roctx through
    ``torch.cuda.nvtx``; the reference brackets the same places with NVTX,
    ``scatter_accumulate.py:307,383,736``), visible to ``rocprofv3 --marker-trace``.

    The reference hops to its comm stream and joins it with the current stream on both sides
    (``gather.py:114,176``; ``scatter_accumulate.py:636-640,725-727``), which orders a launch
    exactly as if it had been issued on the current stream. Here it IS issued on the current
    stream by default: the same ordering without the two event joins per call (35 us of host time
    and about 20 us on the device). ``ODC_COMM_STREAM=dedicated`` restores the hop. With every
    stream at the default priority the hop costs a Llama layer stack nothing measurable (21.6
    against 21.8 ms per microbatch); next to torch FSDP2's own high-priority all-gather and
    reduce-scatter streams the default-priority comm stream cost 30 % (28.2 ms), which is one
    reason why ``patch_fsdp2`` re-creates those streams at the default priority.

    This sits on the host path of every launch, so the default policy asks torch for the raw
    handle of the current stream only (a stream object is built when ``sync`` needs one)."""

    __slots__ = ("label", "cuda_stream", "_traced", "_current", "_comm")

    def __init__(self, label: str = "odc"):
        self.label = label

    def __enter__(self):
        self._traced = _tracing()
        self._comm = None
        if self._traced:
            torch.cuda.nvtx.range_push(self.label)
        try:
            if launch_stream_policy() == "caller":
                handle = _current_raw_stream(get_world().arena.device)
                if handle not in _launch_streams:
                    with _launch_lock:
                        _launch_streams.setdefault(handle, None)
                self.cuda_stream = handle
                return self
            current = torch.cuda.current_stream()
            comm = get_comm_stream()
            with _launch_lock:
                _launch_streams[comm.cuda_stream] = comm
            self.cuda_stream = comm.cuda_stream
            if current == comm:
                return self
            comm.wait_stream(current)
            self._current, self._comm = current, comm
            return self
        except BaseException:
            if self._traced:
                torch.cuda.nvtx.range_pop()
            raise

    def __exit__(self, exc_type, exc, tb):
        try:
            if self._comm is not None:
                self._current.wait_stream(self._comm)
        finally:
            if self._traced:
                torch.cuda.nvtx.range_pop()
        return False


def wait_for_launches() -> None:
    """Block the host until every launch issued through ``comm_stream_section`` has finished."""
    with _launch_lock:
        pending = list(_launch_streams.items())
        _launch_streams.clear()
    for handle, s in pending:
        try:
            (s if s is not None else stream_from_handle(handle)).synchronize()
        except RuntimeError:
            # a stream destroyed since its launch cannot be waited for by name
            torch.cuda.synchronize(get_world().arena.device)


class BufferSplitter:
    """Sub-request sizing rule of the reference (``utils.py:212-242``), in elements.

    ``ODC_MAX_BUFFER_SIZE`` (default 64 Mi elements; <= 0 turns splitting off) caps the staging
    buffer of a whole request; one rank's slice of it is rounded up to 64 elements. Callers size
    buffers with these numbers, so the closed forms are kept; the fused kernels here never
    split a request, and results do not depend on the setting.
    """

    DEFAULT_MAX_BUFFER_SIZE = 64 * 1024 * 1024

    def __init__(self):
        self.round_data_size = 2**6

    def get_max_global_buffer_size(self) -> int:
        return int(os.environ.get("ODC_MAX_BUFFER_SIZE", self.DEFAULT_MAX_BUFFER_SIZE))

    def round_to_data_size(self, size: int) -> int:
        q = self.round_data_size
        return -(-size // q) * q

    def get_global_buffer_size(self, original_buffer_shape) -> int:
        numel = math.prod(original_buffer_shape)
        cap = self.get_max_global_buffer_size()
        return numel if cap <= 0 else min(cap, numel)

    def get_local_buffer_size(self, original_buffer_shape, world_size) -> int:
        numel = math.prod(original_buffer_shape)
        cap = self.get_max_global_buffer_size()
        if cap > 0:
            assert (
                cap % world_size == 0
            ), f"ODC_MAX_BUFFER_SIZE: {cap} % world_size: {world_size} != 0"
            numel = min(cap // world_size, numel)
        return self.round_to_data_size(numel)
