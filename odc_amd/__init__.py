"""odc_amd — MI355X-native gather / scatter-accumulate behind ODC's Python surface.

The reference package exports ``init_nvshmem``, ``SymmBufferRegistry``, ``ReductionService``,
``GatherService`` and ``finalize_distributed`` (``odc/__init__.py:12-18``); the same names are
exported here, so ``import odc_amd as odc`` is the switch. The virtual-world helpers
(``VirtualGroup``, ``set_rank``, ``virtual_rank``, ``get_rank``) come on top.
"""

import logging as _logging

from odc_amd import primitives as _primitives

_EXPORTS = (
    # the reference's surface
    "init_nvshmem", "SymmBufferRegistry", "ReductionService", "GatherService", "finalize_distributed",
    # W virtual ranks in one process
    "VirtualGroup", "set_rank", "virtual_rank", "get_rank",
)
globals().update({name: getattr(_primitives, name) for name in _EXPORTS})
__all__ = list(_EXPORTS)

# silent unless the application configures logging
_logging.getLogger(__name__).addHandler(_logging.NullHandler())
