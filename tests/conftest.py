import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    from oracle import build as obuild

    obuild.build()
    orc.lib()
    return orc


@pytest.fixture(scope="session")
def gpu():
    """torch device for GPU tests; the HIP library must load (no fallback)."""
    import torch

    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    from pie_amd import _lib

    _lib.kernels()
    return torch.device("cuda:0")
