"""inpc_build_cdf_static (the entry point that allocates nothing: its chunk totals live in a scratch array
built into the library) against inpc_build_cdf (caller's workspace) through the C ABI, bit for bit: two calls
in a row on the shared scratch, the second with a smaller input, then the largest size it admits, then the limit."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from inpc_amd import _lib
from tests import helpers as H

pytestmark = pytest.mark.gpu

MAX_LEAVES = 4194304   # INPC_BUILD_CDF_STATIC_MAX_LEAVES


def _static_cdf(w_dev, expect_no_allocation=True):
    lib = _lib.lib()
    n = w_dev.numel()
    cdf = w_dev.clone()
    head = torch.zeros(int(lib.inpc_cdf_head_floats(n)), dtype=torch.float32, device=w_dev.device)
    # free device memory as the driver sees it: an allocation inside the library (which torch's own counters would
    # not show) would lower it. (Under the CPU simulator of tests/cpu_sim there is no such accounting: the
    # comparison of the results is what that run checks.)
    on_gpu = w_dev.device.type == "cuda"
    if on_gpu:
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        before = torch.cuda.memory_allocated()
    _lib.check(lib.inpc_build_cdf_static(_lib.ptr(cdf), _lib.ptr(head), head.numel(), n, H.stream()),
               "inpc_build_cdf_static")
    if on_gpu:
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        if expect_no_allocation:
            assert torch.cuda.mem_get_info()[0] >= free_before
    return cdf, head


def _weights(n, seed):
    rng = np.random.default_rng(seed)
    w = np.exp(rng.normal(0.0, 1.5, size=n)).astype(np.float32)
    w[rng.random(n) < 0.3] = 0.0   # leaves outside the view
    return w


def _compare(n, seed, expect_no_allocation=True):
    w = H.dev(_weights(n, seed))
    cdf_ref, head_ref = H.build_cdf(w)
    cdf, head = _static_cdf(w, expect_no_allocation)
    np.testing.assert_array_equal(cdf.cpu().numpy().view(np.uint32), cdf_ref.cpu().numpy().view(np.uint32))
    np.testing.assert_array_equal(head.cpu().numpy().view(np.uint32), head_ref.cpu().numpy().view(np.uint32))
    assert float(head[0].item()) > 0.0


def test_static_scratch_matches_workspace_variant_on_two_calls_in_a_row(gpu):
    # the first call of a process on a device is the warm-up that looks the scratch array's address up (the runtime
    # may load the code object then); from the second call on the free device memory must not shrink
    _compare(300001, 0, expect_no_allocation=False)
    _compare(4097, 1)   # smaller: stale totals of the first call stay behind it in the scratch
    _compare(300001, 2)


def test_static_scratch_at_its_largest_size(gpu):
    # 4,194,304 leaves are 1024 tiles: 2 x 1024 tile totals + 65536 scanned chunk totals, exactly what the scratch array holds
    _compare(MAX_LEAVES, 3)


def test_static_scratch_rejects_sizes_beyond_its_maximum_and_short_heads(gpu):
    lib = _lib.lib()
    w = torch.zeros(16, dtype=torch.float32, device=gpu)
    head = torch.zeros(int(lib.inpc_cdf_head_floats(MAX_LEAVES + 1)), dtype=torch.float32, device=gpu)
    rc = lib.inpc_build_cdf_static(_lib.ptr(w), _lib.ptr(head), head.numel(), MAX_LEAVES + 1, H.stream())
    assert rc == -3
    assert b"4194304" in lib.inpc_last_error()
    assert lib.inpc_build_cdf_static(None, _lib.ptr(head), head.numel(), 16, H.stream()) == -1
    # a head sized for a small octree is refused for a large one before anything is launched
    small = int(lib.inpc_cdf_head_floats(16))
    assert lib.inpc_build_cdf_static(_lib.ptr(w), _lib.ptr(head), small, 2_097_152, H.stream()) == -2
    assert b"head" in lib.inpc_last_error()
