"""inpc_build_cdf_static (the entry point that allocates nothing: its chunk totals live in a scratch array
built into the library) against inpc_build_cdf (caller's workspace) through the C ABI, bit for bit: two calls
in a row on the shared scratch, the second with a smaller input, then the size limit."""
from __future__ import annotations

import numpy as np
import pytest
import torch

import helpers as H
from inpc_amd import _lib

pytestmark = pytest.mark.gpu


def _static_cdf(w_dev):
    lib = _lib.lib()
    n = w_dev.numel()
    cdf = w_dev.clone()
    head = torch.zeros(int(lib.inpc_cdf_head_floats(n)), dtype=torch.float32, device=w_dev.device)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(lib.inpc_build_cdf_static(_lib.ptr(cdf), _lib.ptr(head), n, H.stream()), "inpc_build_cdf_static")
    assert torch.cuda.memory_allocated() == before
    return cdf, head


def _weights(n, seed):
    rng = np.random.default_rng(seed)
    w = np.exp(rng.normal(0.0, 1.5, size=n)).astype(np.float32)
    w[rng.random(n) < 0.3] = 0.0   # leaves outside the view
    return w


def test_static_scratch_matches_workspace_variant_on_two_calls_in_a_row(gpu):
    for n, seed in ((300001, 0), (4097, 1)):   # the second call is smaller: stale totals of the first stay behind it
        w = H.dev(_weights(n, seed))
        cdf_ref, head_ref = H.build_cdf(w)
        cdf, head = _static_cdf(w)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(cdf.cpu().numpy().view(np.uint32), cdf_ref.cpu().numpy().view(np.uint32))
        np.testing.assert_array_equal(head.cpu().numpy().view(np.uint32), head_ref.cpu().numpy().view(np.uint32))
        assert float(head[0].item()) > 0.0


def test_static_scratch_rejects_sizes_beyond_its_maximum(gpu):
    lib = _lib.lib()
    w = torch.zeros(16, dtype=torch.float32, device="cuda:0")
    head = torch.zeros(_lib.CDF_HEAD_FLOATS, dtype=torch.float32, device="cuda:0")
    rc = lib.inpc_build_cdf_static(_lib.ptr(w), _lib.ptr(head), 4194304 + 1, H.stream())
    assert rc == -3
    assert b"4194304" in lib.inpc_last_error()
    assert lib.inpc_build_cdf_static(None, _lib.ptr(head), 16, H.stream()) == -1
