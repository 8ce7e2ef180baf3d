"""Copies of the sharded parameters in the compute dtype, for the two FSDP modules."""

from __future__ import annotations

from typing import Sequence

import torch

from odc_amd.primitives.utils import SymmBufferRegistry

_epoch = 0  # bumped by the minibatch hooks: the sharded parameters may have changed since


def shards_may_have_changed() -> None:
    """Every copy made so far counts as out of date: the next gather converts anew. Called by the
    minibatch hooks and by everything in this package that rewrites shards; call it after writing
    sharded parameters in a way torch's version counters do not see."""
    global _epoch
    _epoch += 1


def compute_dtype_shards_of(gather_service, src_key, numel: int, dtype: torch.dtype,
                            watch: Sequence[torch.Tensor] = ()) -> torch.Tensor:
    """The symmetric buffer ``src_key`` (a group's sharded parameters, ``numel`` elements per
    rank) converted to ``dtype``, as a second symmetric buffer that is brought up to date before
    it is returned: the calling rank's view of it, to gather from instead of converting on the way.

    The reference gathers the fp32 shards and casts afterwards (fsdp2.py:341-343,
    fsdp1.py:199-223); the fused gather here converts on the way (4 + 2 bytes per element and
    gather). With this copy a gather moves 2 + 2 bytes per element, and the conversion (4 + 2
    bytes per element of the shards) is paid once per change of the shards instead of twice per
    microbatch. It costs the copy's memory: ``numel`` elements of ``dtype`` per rank.

    The copy counts as out of date when a minibatch hook ran since it was made
    (``pre_minibatch_start``, ``pre_optimizer_step`` of either FSDP module: the optimizer step lies
    between them), or when torch has written to the shards since: the version counters of every rank's source
    buffer (writes through views of it: ``fill_peer_shards``, ``load_full_params``) and of the
    tensors in ``watch`` — the sharded parameters themselves, whose in-place updates as DTensors
    (optimizers, ``load_state_dict``) bump the DTensor's counter, not its local tensor's. Writes
    that no version counter sees need ``shards_may_have_changed()`` afterwards (exported as
    ``odc_amd.fsdp.shards_may_have_changed``): ``param.data.copy_()`` and other ``.data`` aliases
    (a detached alias has a counter of its own), tensors built separately over the same memory
    (``arena.view``, ``get_same_node_tensors``), raw pointers. ``fill_peer_shards``,
    ``ParamGroup.load_full_params`` and the ``load_state_dict`` post hook of patched
    ``fully_shard`` modules call it themselves. The bookkeeping lives on the registry, so it ends
    with the arena."""
    registry = SymmBufferRegistry.get_instance()
    key = f"{src_key}_as_{str(dtype).rsplit('.', 1)[-1]}"
    made = registry.__dict__.setdefault("_odc_compute_dtype_shards", {})
    if not registry.has_key(key):
        registry.allocate_symm_buffer(key, (numel,), dtype)
        made.pop(key, None)  # whatever an earlier arena held under this name is gone
    try:
        versions = tuple(t._version for t in (*registry.peer_tensors[src_key], *watch))
    except RuntimeError:  # inference tensors carry no version counter: convert every time
        versions = None
    stamp = (versions, _epoch)
    if versions is None or made.get(key) != stamp:
        gather_service.convert_symm_buffer(key, src_key)
        made[key] = stamp
    return registry.get_symm_buffer(key)
