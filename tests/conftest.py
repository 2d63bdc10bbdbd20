import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (built on demand with g++)."""
    from oracle import oracle as O

    O.lib()
    return O


@pytest.fixture(scope="session")
def gpu():
    """Device handle for GPU tests; fails (not skips) when the HIP library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from inpc_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")
