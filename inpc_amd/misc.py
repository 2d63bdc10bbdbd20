"""Element-wise operators around the appearance field and the loss.

`spherical_contraction`, `compute_normalized_weight_decay_grads`, `add_normalized_weight_decay_grads` and
`fused_cauchy_loss` have the signatures of the reference's (B/torch_bindings/misc.py:9-44);
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


def compute_normalized_weight_decay_grads(weights: torch.Tensor) -> torch.Tensor:
    """Per-level normalised weight-decay gradient of the flat hash-grid parameter vector."""
    weights = _require_gpu_float(weights)
    grads = torch.empty(weights.shape[0], dtype=torch.float32, device=weights.device)
    _lib.check(_lib.lib().inpc_weight_decay_grads(_lib.ptr(weights), _lib.ptr(grads), weights.shape[0], 0,
                                                  _lib.current_stream()), "inpc_weight_decay_grads")
    return grads


def add_normalized_weight_decay_grads(param: torch.nn.Parameter) -> None:
    """param.grad += the same gradient, in place."""
    if param.grad is None:
        raise RuntimeError("the parameter has no gradient to add to")
    if param.data.dtype != torch.float32 or param.grad.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if not (param.data.is_cuda and param.grad.is_cuda and param.data.is_contiguous() and param.grad.is_contiguous()):
        raise RuntimeError("expected contiguous tensors on the GPU")
    _lib.check(_lib.lib().inpc_weight_decay_grads(_lib.ptr(param.data), _lib.ptr(param.grad), param.data.shape[0], 1,
                                                  _lib.current_stream()), "inpc_weight_decay_grads")


class _CauchyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx: Any, input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        input, target = _require_gpu_float(input), _require_gpu_float(target)
        elementwise = torch.empty_like(input)
        _lib.check(_lib.lib().inpc_cauchy_loss(_lib.ptr(input), _lib.ptr(target), _lib.ptr(elementwise), input.numel(),
                                               _lib.current_stream()), "inpc_cauchy_loss")
        ctx.save_for_backward(input, target)
        ctx.set_materialize_grads(False)
        return elementwise.sum()

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad: torch.Tensor):
        input, target = ctx.saved_tensors
        if grad is None:
            return None, None
        grad = _require_gpu_float(grad.reshape(1))
        grad_input = torch.empty_like(input)
        _lib.check(_lib.lib().inpc_cauchy_loss_backward(_lib.ptr(grad), _lib.ptr(input), _lib.ptr(target),
                                                        _lib.ptr(grad_input), input.numel(), _lib.current_stream()),
                   "inpc_cauchy_loss_backward")
        return grad_input, None


def fused_cauchy_loss(input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    """Cauchy loss between input and target with mean reduction."""
    if input.shape != target.shape:
        raise ValueError(f"input and target shapes must match ({input.shape} vs. {target.shape})")
    return _CauchyLoss.apply(input, target)
