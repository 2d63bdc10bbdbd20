"""Element-wise operators between the sampler and the rasterizer.

`spherical_contraction` has the signature of the reference's (B/torch_bindings/misc.py:17-18);
`feature_to_opacity` that of utils.py:31-33, including its gradient (TruncExp, utils.py:13-28).
"""
from __future__ import annotations

from typing import Any

import torch
from torch.autograd.function import once_differentiable

from . import _lib


def _require_gpu_float(t: torch.Tensor) -> torch.Tensor:
    t = t.contiguous()
    if t.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if not t.is_cuda:
        raise RuntimeError("expected tensors on the GPU")
    return t


def spherical_contraction(positions: torch.Tensor) -> torch.Tensor:
    """(N,3) world positions -> (N,3) positions in the unit cube (no gradient, as in the reference)."""
    positions = _require_gpu_float(positions)
    n = positions.shape[0]
    out = torch.empty((n, 3), dtype=torch.float32, device=positions.device)
    _lib.check(_lib.lib().inpc_spherical_contraction(_lib.ptr(positions), _lib.ptr(out), n, _lib.current_stream()),
               "inpc_spherical_contraction")
    return out


class _FeatureToOpacity(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, features: torch.Tensor) -> torch.Tensor:
        features = _require_gpu_float(features.float())
        out = torch.empty_like(features)
        _lib.check(_lib.lib().inpc_opacity_forward(_lib.ptr(features), _lib.ptr(out), features.numel(),
                                                   _lib.current_stream()), "inpc_opacity_forward")
        ctx.save_for_backward(features)
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad: torch.Tensor) -> torch.Tensor:
        (features,) = ctx.saved_tensors
        grad = _require_gpu_float(grad)
        out = torch.empty_like(features)
        _lib.check(_lib.lib().inpc_opacity_backward(_lib.ptr(grad), _lib.ptr(features), _lib.ptr(out), features.numel(),
                                                    _lib.current_stream()), "inpc_opacity_backward")
        return out


def feature_to_opacity(features: torch.Tensor) -> torch.Tensor:
    """Log-space volume density -> opacity in [0, 1]; differentiable."""
    return _FeatureToOpacity.apply(features)
