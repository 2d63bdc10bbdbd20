"""Probability-field statistics update: the per-iteration step that feeds the sampler's leaf indices and the
rasterizer's blending weights back into the octree (Modules/ProbabilityField.py:146-157 of the reference).

`update_probability_field(leaf_weights, leaf_subdivision_scores, indices, weights)` does in place what
`ProbabilityField.update(indices, weights)` does to its two leaf tensors.
"""
from __future__ import annotations

import torch

from . import _lib

#: decay the reference applies to both leaf tensors before the maxima (ProbabilityField.py:149-150)
DECAY = 0.9968


@torch.no_grad()
def update_probability_field(leaf_weights: torch.Tensor, leaf_subdivision_scores: torch.Tensor, indices: torch.Tensor,
                             weights: torch.Tensor, decay: float = DECAY, check: bool = False) -> None:
    """In place: both leaf tensors decay, then leaf_weights takes the per-leaf maximum of the sampled weights and
    the subdivision score the clamped spread (max - min) of them. `check=True` synchronises and raises for an
    index outside the leaf range, as the reference's scatter_reduce_ would."""
    if leaf_weights.dtype != torch.float32 or leaf_subdivision_scores.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if indices.dtype != torch.int64:
        raise RuntimeError("expected scalar type Long")
    if not (leaf_weights.is_contiguous() and leaf_subdivision_scores.is_contiguous()):
        raise RuntimeError("leaf tensors must be contiguous (they are updated in place)")
    if leaf_weights.shape != leaf_subdivision_scores.shape or leaf_weights.dim() != 1:
        raise RuntimeError("leaf tensors must be one-dimensional and of equal length")
    weights = weights.squeeze().to(leaf_weights).contiguous()
    indices = indices.contiguous()
    if weights.dim() > 1 or weights.numel() != indices.numel():
        raise RuntimeError("one weight per index expected")
    if not (leaf_weights.is_cuda and leaf_subdivision_scores.is_cuda and indices.is_cuda and weights.is_cuda):
        raise RuntimeError("expected tensors on the GPU")
    lib = _lib.lib()
    n_leaves = leaf_weights.numel()
    ws_bytes = int(lib.inpc_field_update_workspace_bytes(n_leaves))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=leaf_weights.device)
    stream = _lib.current_stream()
    _lib.check(lib.inpc_field_update(_lib.ptr(indices), _lib.ptr(weights), indices.numel(), _lib.ptr(leaf_weights),
                                     _lib.ptr(leaf_subdivision_scores), n_leaves, float(decay), _lib.ptr(ws), ws_bytes,
                                     stream), "inpc_field_update")
    if check:
        _lib.check(lib.inpc_field_update_check(_lib.ptr(ws), stream), "inpc_field_update")
