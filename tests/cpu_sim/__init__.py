"""A SIMT simulator for the library's own kernels, for tests that have no GPU (TEST INFRASTRUCTURE ONLY).

tests/cpu_sim/build.py compiles inpc_amd/csrc/*.hip, unchanged, with a host compiler (clang++ or g++) against a
stand-in for the HIP runtime (tests/cpu_sim/hip/hip_runtime.h): every thread of a block is a fiber, a wave's
cross-lane operations and a block's barriers are meeting points where the fibers exchange values, blocks run one after
the other (each starting with its LDS filled with a byte pattern), and device memory is host memory. The result,
libinpc_sim.so, exports the same C ABI as the product's library. `simulated_device()` makes it the library that
inpc_amd._lib hands out and "cpu" the device the test helpers allocate on, for as long as the context lasts.

What the simulator shows: the kernels' indexing, their arithmetic (up to the host compiler's and libm's rounding of
exp/log/rsqrt, which the tolerances of the tests cover) and their use of barriers, ballots, shuffles, DPP moves and
atomics. What it cannot show: timing, anything that depends on how the hardware schedules waves of different
blocks (blocks run to completion in order), memory ordering between blocks, register or LDS limits."""
from __future__ import annotations

import contextlib
import ctypes as C
import os


def _aligned_bytes(n_bytes, device):
    import torch

    raw = torch.empty(int(n_bytes) + 256, dtype=torch.uint8, device=device)
    skip = (-raw.data_ptr()) % 256
    return raw[skip:skip + int(n_bytes)]


@contextlib.contextmanager
def simulated_device():
    """Loads libinpc_sim.so in place of libinpc_hip.so. Yields torch.device("cpu")."""
    import torch

    from inpc_amd import _lib, rasterization
    from tests import helpers
    from tests.cpu_sim import build

    path = build.build(sanitize=os.environ.get("INPC_SIM_SANITIZE", "") not in ("", "0"))
    saved = (_lib._lib, _lib.LIB_PATH, _lib.current_stream, helpers.DEVICE, rasterization._new_workspace)
    _lib._lib, _lib.LIB_PATH = None, path
    _lib.current_stream = lambda: C.c_void_p(None)
    helpers.DEVICE = "cpu"
    # a GPU allocation is 256-byte aligned and the rasterizer's workspace relies on it; a host allocation is not
    rasterization._new_workspace = _aligned_bytes
    # the operator layer refuses host tensors; here host memory is the device's
    torch.Tensor.is_cuda = property(lambda self: True)
    try:
        _lib.lib()
        yield torch.device("cpu")
    finally:
        del torch.Tensor.is_cuda
        (_lib._lib, _lib.LIB_PATH, _lib.current_stream, helpers.DEVICE, rasterization._new_workspace) = saved
