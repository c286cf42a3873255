import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_pool():
    """One physical chunk pool for the whole GPU test session (8 GiB of 2 MiB chunks)."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    torch.cuda.set_device(0)
    from glake_amd import vmm_allocator as vmm

    vmm.init_physical_handle(4096, 0)
    yield vmm
