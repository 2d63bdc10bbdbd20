"""Sampler operator API: `compute_viewpoint_weights` and `ProbabilityFieldSampler`.

Same names, arguments and error behaviour as B/torch_bindings/sampling.py:9-132; the native side is
libinpc_hip.so instead of the pybind11 module `_C`.

Differences a caller can observe, all inside what the reference leaves to scheduling:
  * `generate_training_samples` returns the first `n_samples` accepted candidates of the sampler's
    counter-based stream in candidate order (the reference's per-thread streams and atomic slot order
    make both order and multiset run dependent);
  * the generator lives in device memory, so only the calls whose output shape depends on device
    results synchronise the host.
"""
from __future__ import annotations

import ctypes as C
import logging

import torch

from . import _lib
from .views import is_perspective

_log = logging.getLogger("inpc_amd")


def _check_view(view) -> None:
    if not is_perspective(view.camera):
        raise NotImplementedError
    if getattr(view.camera, "distortion", None) is not None:
        raise NotImplementedError


def _prep(centers, levels, weights, view):
    centers = centers.contiguous()
    levels = levels.contiguous()
    weights = weights.contiguous()
    w2c = view.w2c.contiguous()
    if centers.dtype != torch.float32 or weights.dtype != torch.float32 or w2c.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if levels.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int")
    if not (centers.is_cuda and levels.is_cuda and weights.is_cuda and w2c.is_cuda):
        raise RuntimeError("expected tensors on the GPU")
    return centers, levels, weights, w2c


def compute_viewpoint_weights(centers: torch.Tensor, levels: torch.Tensor, weights: torch.Tensor, view,
                              initial_size: float) -> torch.Tensor:
    """Per-leaf view-dependent weight (B/torch_bindings/sampling.py:9-34)."""
    _check_view(view)
    centers, levels, weights, w2c = _prep(centers, levels, weights, view)
    n = centers.shape[0]
    out = torch.empty(n, dtype=torch.float32, device=centers.device)
    cam = _lib.make_camera(view.camera)
    _lib.check(_lib.lib().inpc_leaf_weights(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(w2c),
                                            _lib.ptr(out), None, n, C.byref(cam), float(initial_size),
                                            _lib.current_stream()), "inpc_leaf_weights")
    return out


class ProbabilityFieldSampler(torch.nn.Module):
    """Counterpart of B/torch_bindings/sampling.py:37-132 + ProbabilityFieldSampler of
    B/sampling/include/sampling_api.h:26-82 (generator constructed as pcg32(seed), stream 1)."""

    #: candidates drawn in the first round per requested sample, on top of the running estimate
    OVERSAMPLE = 1.02

    def __init__(self, seed: int) -> None:
        super().__init__()
        host = (C.c_uint64 * 2)()
        _lib.lib().inpc_pcg32_seed(host, C.c_uint64(int(seed) & (2**64 - 1)), C.c_uint64(1))
        self._rng_host_init = (int(host[0]), int(host[1]))
        self._rng = None  # device tensor, created on first use (on the inputs' device)
        self._acceptance = 1.0
        self.last_consumed = 0

    # -- generator ------------------------------------------------------------------------------------
    def _rng_dev(self, device) -> torch.Tensor:
        if self._rng is None or self._rng.device != device:
            state, inc = self._rng_host_init
            signed = [v - 2**64 if v >= 2**63 else v for v in (state, inc)]
            self._rng = torch.tensor(signed, dtype=torch.int64, device=device)
        return self._rng

    def rng_state(self) -> tuple[int, int]:
        """{state, inc} of the generator as unsigned integers (synchronises)."""
        if self._rng is None:
            return self._rng_host_init
        s, i = self._rng.cpu().tolist()
        return s % 2**64, i % 2**64

    # -- shared front end: leaf weights -> CDF -----------------------------------------------------------
    def _weights(self, centers, levels, weights, w2c, view, initial_size):
        n = centers.shape[0]
        lib = _lib.lib()
        stream = _lib.current_stream()
        cam = _lib.make_camera(view.camera)
        vw = torch.empty(max(n, 1), dtype=torch.float32, device=centers.device)
        boxes = torch.empty((max(n, 1), 4), dtype=torch.float32, device=centers.device)  # centre, edge length
        _lib.check(lib.inpc_leaf_weights(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(w2c),
                                         _lib.ptr(vw), _lib.ptr(boxes), n, C.byref(cam), float(initial_size), stream),
                   "inpc_leaf_weights")
        ws_bytes = int(lib.inpc_sampler_workspace_bytes(max(n, 1)))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=centers.device)
        head_floats = int(lib.inpc_cdf_head_floats(max(n, 1)))
        # CDF head; [0] = total, written by inpc_build_cdf / inpc_expected_counts whenever there are leaves
        total = (torch.empty if n > 0 else torch.zeros)(head_floats, dtype=torch.float32, device=centers.device)
        return vw, boxes, ws, ws_bytes, total, cam, stream

    def _cdf(self, centers, levels, weights, w2c, view, initial_size):
        vw, boxes, ws, ws_bytes, total, cam, stream = self._weights(centers, levels, weights, w2c, view, initial_size)
        n = centers.shape[0]
        if n > 0:
            _lib.check(_lib.lib().inpc_build_cdf(_lib.ptr(vw), _lib.ptr(total), total.numel(), _lib.ptr(ws), ws_bytes, n,
                                                 stream), "inpc_build_cdf")
        return vw, boxes, total, cam, stream

    # -- API ---------------------------------------------------------------------------------------------
    def generate_training_samples(self, centers, levels, weights, view, n_samples: int,
                                  initial_size: float) -> tuple[torch.Tensor, torch.Tensor]:
        """(positions (n,3) f32, leaf indices (n,) i64), every position inside the view frustum
        (B/torch_bindings/sampling.py:42-70; B/sampling/src/sampling.cu:50-148)."""
        _check_view(view)
        centers, levels, weights, w2c = _prep(centers, levels, weights, view)
        lib = _lib.lib()
        device = centers.device
        n_leaves = centers.shape[0]
        n_samples = int(n_samples)
        positions = torch.empty((n_samples, 3), dtype=torch.float32, device=device)
        ids64 = torch.empty(n_samples, dtype=torch.int64, device=device)   # written by the kernels as int64
        if n_samples == 0:
            return positions, ids64
        if n_leaves == 0:
            positions.zero_()
            ids64.fill_(-1)
            return positions, ids64
        cdf, boxes, total, cam, stream = self._cdf(centers, levels, weights, w2c, view, initial_size)
        rng = self._rng_dev(device)
        first = min(int(n_samples / max(self._acceptance, 1e-3) * self.OVERSAMPLE) + 4096, (1 << 30) - 1)
        cull_bytes = int(lib.inpc_cull_workspace_bytes(first))
        cull_ws = torch.empty(cull_bytes, dtype=torch.uint8, device=device)
        k0, accepted, consumed = 0, C.c_uint32(0), C.c_uint32(0)
        n_round = first
        finished = False

        def finish(total_candidates):
            _lib.check(lib.inpc_cull_finish(_lib.ptr(total), _lib.ptr(positions), _lib.ptr(ids64), 1, n_samples,
                                            total_candidates, _lib.ptr(rng), _lib.ptr(cull_ws), cull_bytes, stream),
                       "inpc_cull_finish")

        while True:
            _lib.check(lib.inpc_sample_cull_compact(_lib.ptr(boxes), _lib.ptr(cdf), _lib.ptr(total), total.numel(),
                                                    _lib.ptr(w2c), _lib.ptr(positions), _lib.ptr(ids64), 1, n_samples,
                                                    k0, n_round, n_leaves, C.byref(cam), _lib.ptr(rng),
                                                    _lib.ptr(cull_ws), cull_bytes, stream), "inpc_sample_cull_compact")
            k0 += n_round
            if k0 == n_round:
                # the first round nearly always completes the draw: its end is enqueued before the counts are read
                # back, so the device does not wait for the host's round trip (it changes nothing if more rounds follow)
                finish(_lib.CULL_IF_COMPLETE)
            _lib.check(lib.inpc_cull_read_counts(_lib.ptr(cull_ws), C.byref(accepted), C.byref(consumed), stream),
                       "inpc_cull_read_counts")
            finished = k0 == n_round and consumed.value != 0
            if consumed.value != 0 or accepted.value >= n_samples:
                break
            if accepted.value == 0 and k0 >= first:
                # nothing accepted at all: either the weight sum is not positive (failure pattern
                # below) or the frustum is never hit; stop instead of looping forever
                break
            rate = max(accepted.value / k0, 1e-3)
            n_round = min(int((n_samples - accepted.value) / rate * 1.1) + 4096, first)
            if k0 + n_round >= (1 << 30):
                break
        if consumed.value:
            self._acceptance = n_samples / consumed.value
        self.last_consumed = int(consumed.value) if consumed.value else k0
        if not finished:
            finish(k0)
        if consumed.value == 0 and accepted.value < n_samples and float(total[0].item()) > 0.0:
            # the draw gave up (the frustum is hardly ever hit, or the candidate limit was reached): the slots behind
            # the accepted samples get the failure pattern of B/sampling/src/sampling.cu:107-111, positions 0 and
            # index -1, instead of whatever the buffers held (the reference's kernel would not return here)
            _log.warning("sampler accepted only %d of %d samples; the rest is filled with position 0 / index -1",
                         accepted.value, n_samples)
            positions[accepted.value:].zero_()
            ids64[accepted.value:].fill_(-1)
        return positions, ids64

    def generate_samples(self, centers, levels, weights, view, n_samples: int, initial_size: float) -> torch.Tensor:
        """positions (n,3) f32, no culling; an empty (0,3) tensor when no leaf is visible
        (B/torch_bindings/sampling.py:72-100; B/sampling/src/sampling_api.cu:105-168)."""
        _check_view(view)
        centers, levels, weights, w2c = _prep(centers, levels, weights, view)
        device = centers.device
        n_leaves = centers.shape[0]
        if n_leaves == 0:
            return torch.empty((0, 3), dtype=torch.float32, device=device)
        cdf, boxes, total, cam, stream = self._cdf(centers, levels, weights, w2c, view, initial_size)
        if not float(total[0].item()) > 0.0:  # the reference reads the sum back here as well
            return torch.empty((0, 3), dtype=torch.float32, device=device)
        n_samples = int(n_samples)
        positions = torch.empty((n_samples, 3), dtype=torch.float32, device=device)
        _lib.check(_lib.lib().inpc_sample(_lib.ptr(boxes), _lib.ptr(cdf), _lib.ptr(total), total.numel(),
                                          _lib.ptr(positions), None, n_samples, n_leaves,
                                          _lib.ptr(self._rng_dev(device)), stream), "inpc_sample")
        return positions

    def generate_expected_samples(self, centers, levels, weights, view, n_samples: int, n_multi: int,
                                  initial_size: float) -> torch.Tensor:
        """positions (n_created*n_multi, 3) f32 (B/torch_bindings/sampling.py:102-132;
        B/sampling/src/sampling_api.cu:170-240)."""
        _check_view(view)
        centers, levels, weights, w2c = _prep(centers, levels, weights, view)
        lib = _lib.lib()
        device = centers.device
        n_leaves = centers.shape[0]
        if n_leaves == 0:
            return torch.empty((0, 3), dtype=torch.float32, device=device)
        vw, _, ws, ws_bytes, total, cam, stream = self._weights(centers, levels, weights, w2c, view, initial_size)
        offsets = torch.empty(n_leaves, dtype=torch.int32, device=device)
        _lib.check(lib.inpc_expected_counts(_lib.ptr(vw), _lib.ptr(total), _lib.ptr(offsets), int(n_samples),
                                            _lib.ptr(ws), ws_bytes, n_leaves, stream), "inpc_expected_counts")
        n_created = int(offsets[-1].item())  # shape of the result depends on it, as in the reference
        if n_created <= 0:
            return torch.empty((0, 3), dtype=torch.float32, device=device)
        n_total = n_created * int(n_multi)
        ids = torch.empty(n_created, dtype=torch.int32, device=device)
        positions = torch.empty((n_total, 3), dtype=torch.float32, device=device)
        _lib.check(lib.inpc_expected_samples(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(offsets), _lib.ptr(ids),
                                             _lib.ptr(positions), n_created, int(n_multi), n_leaves,
                                             float(initial_size), _lib.ptr(self._rng_dev(device)), stream),
                   "inpc_expected_samples")
        return positions
