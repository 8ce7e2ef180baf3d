"""Minibatch hooks and call-site glue for torch FSDP1 / FSDP2 on top of the primitives.

``shards_may_have_changed()`` is the one call user code may need from here: with
``compute_dtype_shards`` on, it tells both FSDP modules that the sharded parameters were written
in a way torch's version counters do not see (``param.data.copy_()``, raw pointers), so the copies
kept in the compute dtype are converted anew before the next gather.
"""

from odc_amd.fsdp.shard_copies import shards_may_have_changed

__all__ = ["shards_may_have_changed"]
