import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def make_world():
    """Factory: make_world(W, bytes_per_rank) -> VirtualGroup; everything is torn down after
    the test (registry, arena, comm stream)."""
    import torch

    from odc_amd.primitives import utils

    created = []

    def _make(world_size, symmetric_size):
        assert torch.cuda.is_available(), "GPU test run without a GPU"
        group = utils.init_nvshmem(world_size=world_size, symmetric_size=symmetric_size)
        created.append(group)
        return group

    yield _make
    from odc_amd.fsdp import fsdp1, fsdp2

    fsdp1.unpatch_fsdp1()
    fsdp2.unpatch_fsdp2()
    if utils.is_initialized():
        torch.cuda.synchronize()
        utils.SymmBufferRegistry.get_instance().finalize()
        utils.finalize_distributed()
