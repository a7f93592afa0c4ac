import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


def pytest_sessionstart(session):
    """The tests load what has been built; only if no library is there do they build it (the
    product itself never builds or falls back: int4linear_amd._lib.load raises)."""
    from int4linear_amd import _lib

    if not _lib.LIB_PATH.exists():
        from int4linear_amd.build import build_library

        build_library()


@pytest.fixture(scope="session")
def gpu():
    """Device handle for GPU tests; fails (not skips) if the HIP library is missing."""
    import torch

    assert torch.cuda.is_available(), "GPU test selected but no HIP device is visible"
    import int4linear_amd

    int4linear_amd.init()
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def host_threads():
    return max(1, min(16, os.cpu_count() or 1))
