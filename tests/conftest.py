import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_addoption(parser):
    parser.addoption("--sim", action="store_true", default=False,
                     help="run the tests marked gpu on the CPU: the `gpu` fixture loads the kernels compiled for the "
                          "SIMT simulator of tests/cpu_sim instead of the HIP library (use with -m gpu; tests that "
                          "need streams, graphs or the device's memory accounting skip themselves)")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "real_gpu: a gpu test that the simulator of tests/cpu_sim cannot run")


def pytest_collection_modifyitems(config, items):
    if not config.getoption("--sim"):
        return
    skip = pytest.mark.skip(reason="needs the real device (streams, graphs, memory accounting or full sizes)")
    for item in items:
        if item.get_closest_marker("real_gpu") is not None:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (built on demand with g++)."""
    from oracle import oracle as O

    O.lib()
    return O


@pytest.fixture(scope="session")
def maker():
    """tests/golden/make_golden.py as a module: the script that wrote the committed fixtures."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_golden", ROOT / "tests" / "golden" / "make_golden.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


@pytest.fixture(scope="session")
def gpu(request):
    """Device handle for GPU tests; fails (not skips) when the HIP library is missing. With --sim: the CPU, with
    the simulator's build of the kernels loaded in the HIP library's place."""
    import torch

    if request.config.getoption("--sim"):
        from tests.cpu_sim import simulated_device

        with simulated_device() as device:
            yield device
        return
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from inpc_amd import _lib

    _lib.lib()
    yield torch.device("cuda:0")


@pytest.fixture(scope="module")
def sim():
    """The CPU as the device, with the simulator's build of the kernels loaded (tests/cpu_sim): for tests that are
    not marked gpu and run the library's kernels all the same."""
    from tests.cpu_sim import simulated_device

    with simulated_device() as device:
        yield device
