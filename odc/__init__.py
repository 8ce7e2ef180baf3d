"""``odc`` — the reference's import paths, resolved to the ``odc_amd`` modules.

Code written against the reference imports by module path: ``from odc.primitives.gather import
GatherService``, ``from odc.primitives.utils import SymmBufferRegistry, init_nvshmem``
(examples/all_gather.py:10-11), ``from odc.primitives.scatter_accumulate import ReductionService``
(examples/reduce_scatter.py:9-10), ``from odc.fsdp import fsdp2`` and ``from odc import
init_nvshmem`` (examples/FSDP2/example.py:15-17). This package holds no logic: it registers the
``odc_amd`` modules under those names, so the same import lines give the same objects.

The NVSHMEM device externs that ``odc.primitives`` also exports in the reference
(``NVSHMEM_EXTERN_LIBS``, ``putmem_nbi_block``, ``quiet`` ...) belong to its Triton inter-node
kernels, which have no counterpart on one GPU; importing them fails here, as any missing name does.
"""

import importlib as _importlib
import sys as _sys

import odc_amd as _odc_amd

_SUBMODULES = (
    "primitives",
    "primitives.gather",
    "primitives.scatter_accumulate",
    "primitives.utils",
    "primitives.tensor_ipc",
    "fsdp",
    "fsdp.fsdp1",
    "fsdp.fsdp2",
)
for _name in _SUBMODULES:
    _sys.modules[f"{__name__}.{_name}"] = _importlib.import_module(f"odc_amd.{_name}")

primitives = _sys.modules[f"{__name__}.primitives"]
fsdp = _sys.modules[f"{__name__}.fsdp"]

# the package-level names of odc/__init__.py:12-18 (and the virtual-world helpers next to them)
globals().update({_name: getattr(_odc_amd, _name) for _name in _odc_amd.__all__})
__all__ = list(_odc_amd.__all__)
