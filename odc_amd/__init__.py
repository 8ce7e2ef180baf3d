"""odc_amd — MI355X-native gather / scatter-accumulate behind ODC's Python surface.

Same top-level names as the reference package (``odc/__init__.py:12-18``), so
``import odc_amd as odc`` is the switch.
"""

import logging

from odc_amd.primitives.gather import GatherService
from odc_amd.primitives.scatter_accumulate import ReductionService
from odc_amd.primitives.utils import (
    SymmBufferRegistry,
    VirtualGroup,
    finalize_distributed,
    init_nvshmem,
    set_rank,
    virtual_rank,
)

logger = logging.getLogger(__name__)
logger.addHandler(logging.NullHandler())
logger.setLevel(logging.INFO)

__all__ = [
    "init_nvshmem",
    "SymmBufferRegistry",
    "ReductionService",
    "GatherService",
    "finalize_distributed",
    "VirtualGroup",
    "set_rank",
    "virtual_rank",
]
