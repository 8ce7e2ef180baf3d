"""On-demand scatter-accumulate: a full gradient is added, chunk r into rank r's accumulation
buffer, by one fused HIP launch.

Mirror of ``odc/primitives/scatter_accumulate.py`` (``ReductionService``, :494-749). In the
reference the caller copies chunk r into a staging buffer on rank r (:649-669), rings a doorbell
(:671-688) and a watcher process on rank r performs ``acc[start:start+size].add_(buf[:size])``
(:369-395). With every rank's accumulation in one HBM the owner is the caller, so staging,
doorbells and the watcher collapse into ``odc_scatter_accumulate`` (include/odc_hip.h): one read
of the gradient, one read-modify-write of the accumulations.

Clears are eager by default, as in the reference: ``clear_accumulations`` zeroes every
accumulation with one launch. ``ReductionService(lazy_clear=True)`` or ``ODC_LAZY_CLEAR=1`` makes
them lazy: ``clear_accumulations`` then only notes that every accumulation counts as zero, and the
first scatter-accumulate of a key after it runs as ``odc_scatter_store`` (``acc = +0 + grad``, the
accumulation is written but never read). The bits are those of a clear followed by an accumulate;
per minibatch it saves the clear's 4 bytes per element and the first read of the accumulation
(4 more). Whatever hands an accumulation out (``accumulations``, ``get_accumulation``,
``get_peer_accumulations``, ``publish``) first writes the zeros that are still owed; a tensor kept
from an earlier call is not tracked and, in lazy mode only, shows the previous minibatch's sums
between a clear and the next accumulate.

Launch plans are cached: the ctypes item array of a call (accumulation offsets, shard sizes) is
built the first time a list of keys and sizes is seen, per host thread, and later calls only
rewrite the gradient pointers (the reference caches per key too, :599-600).

Callers on several host threads and streams. In the reference every add into rank r's
accumulation goes through r's one watcher (:291-310, :386-392), so clients never race on it. Here
the add is a read-modify-write launched on the caller's stream; the service therefore keeps, per
key, the stream that last wrote it, and a launch for that key on another stream first waits for
the previous one (an event record and a stream wait, only when the stream changes). The service's
bookkeeping and its launches run under one lock, so the adds into one key are serialised in the
order the calls took the lock: any order is a valid sum (fp32 addition commutes up to rounding,
the reference's own cross-client order is arrival order), and calls chained by the caller keep
the caller's order bit for bit.
"""

from __future__ import annotations

import collections.abc
import contextlib
import ctypes
import logging
import os
import threading
from typing import Sequence

import torch

from odc_amd import _native
from odc_amd.primitives.utils import (
    BufferSplitter,
    StreamOrder,
    SymmBufferRegistry,
    comm_stream_section,
    wait_for_launches,
    get_rank,
    get_world,
    group_size,
    native_dtype,
)

logger = logging.getLogger(__name__)


class _LiveAccumulations(collections.abc.Sequence):
    """``ReductionService.accumulations``: the calling rank's live accumulation tensors in
    registration order, ``accumulations[accumulation_indices[key]]`` being the buffer of ``key``
    (the list the reference keeps, scatter_accumulate.py:496,554-555, and that its callers
    iterate and index: ``odc/fsdp/fsdp1.py:324``, ``examples/reduce_scatter.py:169``). Entries are
    looked up when read, so they follow the virtual rank the process currently plays, and reading
    one first writes the zeros a lazy clear still owes it."""

    def __init__(self, service):
        self._service = service

    def __len__(self):
        return len(self._service.accumulation_keys)

    def __getitem__(self, index):
        keys = self._service.accumulation_keys[index]
        if isinstance(index, slice):
            return [self._service.get_accumulation(k) for k in keys]
        return self._service.get_accumulation(keys)

    def __iter__(self):
        for key in list(self._service.accumulation_keys):
            yield self._service.get_accumulation(key)

    def __repr__(self):
        return f"<{len(self)} live accumulations>"


class _AccumPlan:
    """The cached part of one scatter-accumulate call: its item array with everything but the
    gradient pointers filled in."""

    __slots__ = ("items", "n", "grad_code", "acc_code", "acc_dtype", "max_numels", "tiles_exactly", "keys",
                 "layout")

    def __init__(self, n):
        self.items = (_native.AccumItem * n)()
        self.n = n


_MIXED = "mixed"


class ReductionService:
    def __init__(self, accumulation_dtype=None, lazy_clear=None):
        self.accumulation_keys = []  # index -> key, in registration order
        self.accumulations = _LiveAccumulations(self)  # index -> the calling rank's live tensor
        self.accumulation_indices = {}
        self.accumulation_dtype = accumulation_dtype
        self.dispatched_tasks = 0
        self.buffer_splitter = BufferSplitter()
        if lazy_clear is None:
            lazy_clear = os.environ.get("ODC_LAZY_CLEAR", "0") == "1"
        self.lazy_clear = bool(lazy_clear)
        self._owed_zero = set()  # keys whose accumulations count as zero but hold stale bytes
        self._captured = set()  # keys ever accumulated under stream capture: always cleared by a kernel
        # key -> what has been written into the accumulation since a kernel last zeroed all of it:
        # None (nothing), one layout of disjoint slices, or _MIXED (anything else). A lazy clear
        # may be folded into a store over slices only while everything outside them is still zero.
        self._written = {}
        self._sliced_keys = set()  # keys ever used through scatter_accumulate_slices
        self._plans = threading.local()  # per host thread: plan key -> _AccumPlan
        # One lock for the bookkeeping above AND the launches it decides: callers come from several
        # host threads (the autograd device thread in backward), and the order of the bookkeeping
        # must be the order of the launches.
        self._lock = threading.RLock()
        self._order = StreamOrder()  # which stream last wrote each accumulation
        # Inside captured_minibatch(): the keys whose captured clear has not been recorded (yet).
        self._capture_scope = None

    # -- registration ---------------------------------------------------------------------
    @staticmethod
    def _acc_key(key):
        return f"rs_accumulation_{key}"

    def register(self, key, output_tensor_shape, grad_dtype, reduction_dtype, pg):
        """Allocate the zero-initialised symmetric accumulation ``rs_accumulation_{key}``
        (scatter_accumulate.py:551-555; the watcher zeroes it at :357-362). No staging buffers
        are created: the fused kernel reads the caller's gradient directly."""
        assert len(output_tensor_shape) == 1
        with self._lock:
            assert key not in self.accumulation_indices
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError(
                    "register accumulation keys before capturing: the zeroing of a new accumulation "
                    "would be recorded into the graph and run on every replay"
                )
            native_dtype(grad_dtype), native_dtype(reduction_dtype)  # reject unsupported dtypes early
            registry = SymmBufferRegistry.get_instance()
            accumulation_key = self._acc_key(key)
            assert not registry.has_key(accumulation_key)
            registry.allocate_symm_buffer(accumulation_key, tuple(output_tensor_shape), reduction_dtype)
            self.accumulation_indices[key] = len(self.accumulation_keys)
            self.accumulation_keys.append(key)
            self._clear_keys([key])  # a one-time cost; the buffer never shows arena leftovers

    def _clear_keys(self, keys):
        """Launch the clear kernel over ``keys`` (caller holds the lock)."""
        keys = list(keys)
        self._owed_zero.difference_update(keys)
        if self._capture_scope and torch.cuda.is_current_stream_capturing():
            self._capture_scope.difference_update(keys)
        if not keys:
            return
        for key in keys:
            self._written[key] = None
        registry = SymmBufferRegistry.get_instance()
        spans = (_native.Span * len(keys))()
        for i, key in enumerate(keys):
            offset, shape, dtype = registry.offsets[self._acc_key(key)]
            spans[i].offset = offset
            spans[i].nbytes = shape[0] * dtype.itemsize
        with comm_stream_section("odc.clear") as comm:
            self._order_after_writers(keys, comm.cuda_stream)
            _native.check(
                _native.load().odc_clear(
                    get_world().arena.handle, spans, len(spans), ctypes.c_void_p(comm.cuda_stream)
                )
            )

    def _order_after_writers(self, keys, stream_handle) -> None:
        """Before a launch that writes ``keys`` on ``stream_handle``: wait for the launches that
        last wrote them on other streams (caller holds the lock; see the module docstring)."""
        if torch.cuda.is_current_stream_capturing():
            return  # a graph runs on the stream it is replayed on: nothing the host could order
        total = len(self.accumulation_keys)
        self._order.before_launch(keys, stream_handle, all_keys=len(keys) == total, total=total)

    def clear_accumulations(self):
        """Zero every registered accumulation of EVERY virtual rank in one launch
        (``acc.fill_(0)`` per key and per process in the reference, :585-587). Idempotent, so
        each virtual rank may call it; like there, no rank may have started the minibatch's
        scatter-accumulates before the last clear.

        Lazy mode launches nothing here, except for keys that a captured HIP graph accumulates
        into: a graph replays the read-modify-write form whatever the host has noted since, so
        those are always cleared by a kernel (captured too, when this call is)."""
        with self._lock:
            if torch.cuda.is_current_stream_capturing():
                if self._capture_scope is not None:
                    # inside captured_minibatch(): the clear is recorded when (and if) it is needed
                    self._check_no_host_owed(self.accumulation_keys)
                    self._capture_scope.update(self.accumulation_keys)
                else:
                    self._clear_keys(self.accumulation_keys)
                return
            if not self.lazy_clear:
                self._clear_keys(self.accumulation_keys)
                return
            self._clear_keys([k for k in self.accumulation_keys if k in self._captured])
            self._owed_zero.update(k for k in self.accumulation_keys if k not in self._captured)

    @contextlib.contextmanager
    def captured_minibatch(self):
        """``with torch.cuda.graph(g), service.captured_minibatch():`` — capture a whole
        minibatch (``clear_accumulations()`` followed by its scatter-accumulates) with the clear
        folded into the first scatter-accumulate of every key: inside this block a captured
        ``clear_accumulations()`` records nothing, the first captured scatter-accumulate of a key
        after it is recorded in the store form (``acc = +0 + grad``: the bits of a clear followed
        by an accumulate, 6 instead of 4 + 10 bytes per element for bf16 into fp32), and the
        clear kernel is recorded only for what needs it: a key that is read, published or
        accumulated through a gapped slice layout before its first whole accumulate, and, when
        the block ends, every key the graph never accumulated into. Both choices are made from
        what the graph itself holds, never from host state, so every replay is a complete
        minibatch whatever ran before it. Works with eager and lazy clears alike; a capture
        that starts while a lazy clear still owes zeros is refused, as always."""
        with self._lock:
            if not torch.cuda.is_current_stream_capturing():
                raise RuntimeError("captured_minibatch() belongs inside torch.cuda.graph(...)")
            if self._capture_scope is not None:
                raise RuntimeError("captured_minibatch() blocks do not nest")
            self._capture_scope = set()
        try:
            yield self
            with self._lock:
                pending = [k for k in self.accumulation_keys if k in self._capture_scope]
                if pending:  # never accumulated in this graph: their clear is still due
                    self._clear_keys(pending)
        finally:
            with self._lock:
                self._capture_scope = None

    def _check_no_host_owed(self, keys):
        owed = [k for k in keys if k in self._owed_zero]
        if owed:
            raise RuntimeError(
                f"captured while {len(owed)} accumulation(s) still owe the zeros of a lazy clear: a "
                "clear recorded here would run on every replay and never now. Read them once "
                "(get_accumulation) or run one eager scatter-accumulate before capturing, or use "
                "eager clears (lazy_clear=False)."
            )

    def _settle(self, keys):
        """Write the zeros still owed to ``keys`` (before anything reads or adds into them)."""
        if self._capture_scope and torch.cuda.is_current_stream_capturing():
            deferred = [k for k in keys if k in self._capture_scope]
            if deferred:
                self._clear_keys(deferred)  # recorded into the graph, in order
        if self._owed_zero:
            owed = [k for k in keys if k in self._owed_zero]
            if owed:
                if torch.cuda.is_current_stream_capturing():
                    self._check_no_host_owed(owed)
                self._clear_keys(owed)

    def _under_capture(self, keys) -> bool:
        """Bookkeeping for a scatter-accumulate issued while the current stream is captured into
        a HIP graph. What the graph records is replayed as recorded, so the choice between the
        store form and the read-modify-write form cannot depend on host state: the
        read-modify-write form is recorded (or, inside ``captured_minibatch()``, the store form
        for a key whose clear was captured just before), and the keys are from now on cleared by
        kernels outside capture."""
        if not torch.cuda.is_current_stream_capturing():
            return False
        self._check_no_host_owed(keys)
        self._captured.update(keys)
        return True

    def forget_captured_graphs(self):
        """Call after destroying every HIP graph that scatter-accumulates into this service's
        keys: lazy clears may then skip the clear kernel for them again."""
        with self._lock:
            self._captured.clear()

    def _launch(self, keys, items, n, grad_code, acc_code, store):
        if not n:
            return
        lib = _native.load()
        entry = lib.odc_scatter_store if store else lib.odc_scatter_accumulate
        with comm_stream_section("odc.scatter_store" if store else "odc.scatter_accumulate") as comm:
            self._order_after_writers(keys, comm.cuda_stream)
            status = entry(
                get_world().arena.handle, items, n, grad_code, acc_code, ctypes.c_void_p(comm.cuda_stream)
            )
        if status:
            _native.check(status)

    def _plan_cache(self):
        cache = getattr(self._plans, "cache", None)
        if cache is None:
            cache = self._plans.cache = {}
        return cache

    # -- the primitive ----------------------------------------------------------------------
    def infer_output_shape(self, input_tensor, pg):
        assert len(input_tensor.shape) == 1
        assert input_tensor.shape[0] % group_size(pg) == 0
        return (input_tensor.shape[0] // group_size(pg),)

    def scatter_accumulate(self, key, input_tensor, pg) -> None:
        """``acc_r[key] += input_tensor.view(W, -1)[r]`` for every rank r."""
        self.scatter_accumulate_multi([key], [input_tensor], pg)

    def _plan_multi(self, keys, input_tensors, pg, valid_numels, W):
        """Validate a (keys, gradients) list once and build its item array."""
        registry = SymmBufferRegistry.get_instance()
        grad_dtype = input_tensors[0].dtype
        plan = _AccumPlan(len(keys))
        plan.keys = tuple(keys)
        acc_dtype = None
        for i, (key, grad) in enumerate(zip(keys, input_tensors)):
            assert grad.dtype == grad_dtype, "one launch takes one gradient dtype"
            if valid_numels is None:
                shard_shape = self.infer_output_shape(grad, pg)
                valid = grad.numel()
            else:
                assert key in self.accumulation_indices, "padded form needs a registered key"
                shard_shape = registry.offsets[self._acc_key(key)][1]
                valid = int(valid_numels[i])
                assert valid <= grad.numel() and valid <= W * shard_shape[0]
            if key not in self.accumulation_indices:
                accum_dtype = (
                    self.accumulation_dtype if self.accumulation_dtype is not None else grad.dtype
                )
                self.register(key, shard_shape, grad.dtype, accum_dtype, pg)
            offset, acc_shape, this_acc_dtype = registry.offsets[self._acc_key(key)]
            assert tuple(acc_shape) == tuple(
                shard_shape
            ), f"key {key}: registered shard {acc_shape}, gradient implies {shard_shape}"
            assert acc_dtype in (None, this_acc_dtype), "one launch takes one accumulation dtype"
            acc_dtype = this_acc_dtype
            plan.items[i].grad_elems = valid
            plan.items[i].acc_offset = offset
            plan.items[i].shard_elems = shard_shape[0]
        plan.grad_code = native_dtype(grad_dtype)
        plan.acc_code = native_dtype(acc_dtype)
        plan.acc_dtype = acc_dtype
        return plan

    def scatter_accumulate_multi(
        self, keys: Sequence, input_tensors: Sequence[torch.Tensor], pg, valid_numels=None
    ) -> None:
        """Multi-tensor form: all (key, gradient) pairs in ONE launch (per 64 pairs).

        ``valid_numels[i]``, when given, says that only the first so many elements of the
        padded gradient i exist at ``input_tensors[i]``; the rest read as +0 (the ``F.pad`` of
        ``odc/fsdp/fsdp1.py:25-38`` without materialising it). Then ``input_tensors[i]`` may be
        shorter than W * shard and the shard size comes from the registered accumulation.
        """
        n = len(keys)
        assert n == len(input_tensors)
        if not n:
            return
        world = get_world()
        W = group_size(pg)
        assert W == world.world_size, f"group size {W} != arena world size {world.world_size}"
        grad_dtype = input_tensors[0].dtype
        numels = tuple(t.numel() for t in input_tensors)
        plan_key = ("multi", world.serial, tuple(keys), numels, grad_dtype,
                    None if valid_numels is None else tuple(int(v) for v in valid_numels))
        cache = self._plan_cache()
        plan = cache.get(plan_key)
        if plan is None:
            plan = cache[plan_key] = self._plan_multi(keys, input_tensors, pg, valid_numels, W)
        items = plan.items
        for i, grad in enumerate(input_tensors):
            assert grad.is_cuda, "scatter-accumulate runs on the GPU only"
            assert grad.dtype == grad_dtype, "one launch takes one gradient dtype"
            assert grad.is_contiguous()
            items[i].grad = grad.data_ptr()

        with self._lock:
            if self._sliced_keys and not self._sliced_keys.isdisjoint(keys):
                for key in keys:  # a whole-key write also fills what lies between a key's slices
                    self._written[key] = _MIXED
            # the keys that count as zero without holding zeros: owed by a lazy clear, or, in a
            # captured minibatch, by the clear captured just before
            zero = self._capture_scope if self._under_capture(keys) else self._owed_zero
            duplicates = len(set(keys)) != n
            if not duplicates and (not zero or zero.isdisjoint(keys)):
                self._launch(keys, items, n, plan.grad_code, plan.acc_code, False)  # the steady state
            else:
                # Keys that still count as zero take the store form (no read of the accumulation).
                # A key listed k times goes into k consecutive launches, so its gradients add up
                # in list order.
                zero = zero or ()
                rounds, times_seen = [], {}
                for i, key in enumerate(keys):
                    k = times_seen.get(key, 0)
                    times_seen[key] = k + 1
                    if k == len(rounds):
                        rounds.append([])
                    rounds[k].append(i)
                for k, members in enumerate(rounds):
                    for store in (True, False):
                        picked = [i for i in members if (k == 0 and keys[i] in zero) == store]
                        if not picked:
                            continue
                        part = (_native.AccumItem * len(picked))(*[items[i] for i in picked])
                        self._launch([keys[i] for i in picked], part, len(picked), plan.grad_code, plan.acc_code,
                                     store)
                if zero:
                    zero.difference_update(keys)
            self.dispatched_tasks += n

    def scatter_accumulate_slices(
        self,
        key,
        input_tensors: Sequence[torch.Tensor],
        slice_offsets: Sequence[int],
        slice_numels: Sequence[int],
        pg,
        accumulation_numel: int = None,
        accumulation_dtype=None,
    ) -> None:
        """Accumulate several gradients into slices of ONE accumulation, in one launch:
        ``acc_r[key][off_i : off_i + n_i] += pad0(input_i).view(W, n_i)[r]``, where ``input_i``
        holds at most ``W * n_i`` elements and what is missing reads as +0.

        With the FSDP2 group layout this is ``torch._chunk_cat`` (``odc/fsdp/fsdp2.py:671-682``)
        followed by ``scatter_accumulate`` (``fsdp2.py:708-710``) without the intermediate
        ``[W, sum n_i]`` reduce-scatter input. The key is registered on first use with
        ``accumulation_numel`` elements (default: the end of the last slice).
        """
        n = len(input_tensors)
        assert n == len(slice_offsets) == len(slice_numels)
        if not n:
            return
        world = get_world()
        W = group_size(pg)
        assert W == world.world_size, f"group size {W} != arena world size {world.world_size}"
        grad_dtype = input_tensors[0].dtype
        plan_key = ("slices", world.serial, key, tuple(slice_offsets), tuple(slice_numels), grad_dtype)
        cache = self._plan_cache()
        plan = cache.get(plan_key)
        if plan is None:
            registry = SymmBufferRegistry.get_instance()
            if key not in self._sliced_keys:
                self._sliced_keys.add(key)
                self._written[key] = _MIXED  # whatever whole-key calls wrote before was not tracked
            if key not in self.accumulation_indices:
                total = accumulation_numel
                if total is None:
                    total = max(o + m for o, m in zip(slice_offsets, slice_numels))
                accum_dtype = accumulation_dtype or self.accumulation_dtype or grad_dtype
                self.register(key, (total,), grad_dtype, accum_dtype, pg)  # zeroes it: nothing written
            offset, acc_shape, acc_dtype = registry.offsets[self._acc_key(key)]
            plan = _AccumPlan(n)
            plan.keys = (key,)
            plan.max_numels = []
            for i, (off, m) in enumerate(zip(slice_offsets, slice_numels)):
                assert 0 <= off and off + m <= acc_shape[0], "slice leaves the accumulation"
                plan.items[i].acc_offset = offset + off * acc_dtype.itemsize
                plan.items[i].shard_elems = m
                plan.max_numels.append(W * m)
            # The store form overwrites the slices and nothing else, so it can stand in for a
            # clear only if the slices are disjoint and the rest of the accumulation holds zeros:
            # either there is no rest (the slices tile the accumulation), or nothing but these
            # very slices has been written since a kernel last zeroed all of it (self._written).
            layout = tuple(sorted((int(o), int(m)) for o, m in zip(slice_offsets, slice_numels) if m))
            end, disjoint, gaps = 0, True, False
            for o, m in layout:
                if o < end:
                    disjoint = False
                    break
                gaps |= o != end
                end = o + m
            plan.layout = layout if disjoint else None
            plan.tiles_exactly = disjoint and not gaps and end == acc_shape[0]
            plan.grad_code = native_dtype(grad_dtype)
            plan.acc_code = native_dtype(acc_dtype)
            plan.acc_dtype = acc_dtype
            cache[plan_key] = plan
        items = plan.items
        for i, grad in enumerate(input_tensors):
            numel = grad.numel()
            assert grad.is_cuda and grad.is_contiguous() and grad.dtype == grad_dtype
            assert numel <= plan.max_numels[i], f"gradient {i} has {numel} > {W} * {slice_numels[i]} elements"
            items[i].grad = grad.data_ptr()
            items[i].grad_elems = numel
        with self._lock:
            store = False
            written = self._written.get(key, _MIXED)
            if self._under_capture(plan.keys):
                # In a captured minibatch the store form stands in for the captured clear only
                # when the slices tile the accumulation: what lies between the slices of a gapped
                # layout at the time of a replay is not known when the graph is recorded.
                if self._capture_scope and key in self._capture_scope:
                    store = plan.tiles_exactly
                    if store:
                        self._capture_scope.discard(key)
                    else:
                        self._settle([key])
                        written = None
            elif key in self._owed_zero:
                store = plan.tiles_exactly or (plan.layout is not None and written in (None, plan.layout))
                if store:
                    self._owed_zero.discard(key)
                else:
                    self._settle([key])
                    written = None
            self._written[key] = plan.layout if plan.layout is not None and written in (None, plan.layout) else _MIXED
            self._launch(plan.keys, items, n, plan.grad_code, plan.acc_code, store)
            self.dispatched_tasks += 1

    # -- results ----------------------------------------------------------------------------
    def get_accumulation(self, key, within_slices: bool = False):
        """The calling rank's live accumulation buffer (callers mutate it in place,
        ``odc/fsdp/fsdp2.py:846-847``). With lazy clears, a tensor kept from an earlier call is
        not updated by ``clear_accumulations`` until the next accumulate; ask again instead.

        ``within_slices=True`` is the caller's promise to write only inside the slices the key
        is accumulated through (``scatter_accumulate_slices``); without it the service assumes
        that the caller may write anywhere in the buffer, also between the slices of a gapped
        layout, and the next lazy clear of the key is a real one."""
        with self._lock:
            if key not in self.accumulation_indices:
                raise KeyError(key)
            self._settle([key])
            self._handed_out([key], within_slices)
            return SymmBufferRegistry.get_instance().get_symm_buffer(self._acc_key(key))

    def _handed_out(self, keys, within_slices):
        """A live accumulation leaves the service: what its holder writes is not tracked, so the
        bytes between the slices of a gapped layout no longer count as zeros."""
        if self._sliced_keys and not within_slices:
            for key in keys:
                if key in self._sliced_keys:
                    self._written[key] = _MIXED

    def publish(self, keys: Sequence, out_dtype=None, divisor: float = 1.0, within_slices: bool = False):
        """End-of-minibatch pass over the calling rank's accumulations ``keys``, in one launch:
        ``acc /= divisor`` in place (skipped for 1) and, when ``out_dtype`` differs from the
        accumulation dtype, a cast copy. Returns one tensor per key: the cast copy, or the live
        accumulation itself when no cast is needed (as ``acc.to(dtype)`` does; ``within_slices``
        as for ``get_accumulation``).
        ``odc/fsdp/fsdp1.py:324-335``; ``odc/fsdp/fsdp2.py:846-847,897-899``."""
        if not keys:
            return []
        with self._lock:
            self._settle(keys)
            registry = SymmBufferRegistry.get_instance()
            items = (_native.PublishItem * len(keys))()
            results, acc_dtype = [], None
            for i, key in enumerate(keys):
                offset, shape, dtype = registry.offsets[self._acc_key(key)]
                assert acc_dtype in (None, dtype), "one launch takes one accumulation dtype"
                acc_dtype = dtype
                acc = registry.get_symm_buffer(self._acc_key(key))
                items[i].acc_offset = offset
                items[i].elems = shape[0]
                if out_dtype is None or out_dtype == dtype:
                    items[i].out = None
                    results.append(acc)
                    self._handed_out([key], within_slices)
                else:
                    out = torch.empty(shape, dtype=out_dtype, device=acc.device)
                    items[i].out = out.data_ptr()
                    results.append(out)
            target = acc_dtype if out_dtype is None else out_dtype
            with comm_stream_section("odc.publish") as comm:
                self._order_after_writers(keys, comm.cuda_stream)
                _native.check(
                    _native.load().odc_publish(
                        get_world().arena.handle,
                        get_rank(),
                        items,
                        len(items),
                        native_dtype(acc_dtype),
                        native_dtype(target),
                        float(divisor),
                        ctypes.c_void_p(comm.cuda_stream),
                    )
                )
        return results

    def accumulation_dtype_of(self, key) -> torch.dtype:
        """The dtype the accumulation of ``key`` was registered with."""
        return SymmBufferRegistry.get_instance().offsets[self._acc_key(key)][2]

    def _registry_peers(self, key):
        """The W accumulation buffers as they are in memory (owed zeros not written)."""
        return SymmBufferRegistry.get_instance().peer_tensors[self._acc_key(key)]

    def get_peer_accumulations(self, key):
        """All W ranks' accumulation buffers for ``key`` (virtual-world convenience)."""
        with self._lock:
            self._settle([key])
            self._handed_out([key], False)
            return SymmBufferRegistry.get_instance().peer_tensors[self._acc_key(key)]

    def sync(self, pg=None):
        """Block until every dispatched add has landed (:734-743: the reference counts tasks
        across ranks and waits for its watcher; here it waits for the streams launched on)."""
        wait_for_launches()
        with self._lock:
            self.dispatched_tasks = 0

    def stop(self):
        if torch.cuda.is_available():
            wait_for_launches()
