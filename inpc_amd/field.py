"""Probability-field bookkeeping: the per-iteration statistics update that feeds the sampler's leaf indices and
the rasterizer's blending weights back into the octree, and the two restructuring steps that follow from it
(Modules/ProbabilityField.py:146-165, 217-257 of the reference).

`update_probability_field(leaf_weights, leaf_subdivision_scores, indices, weights)` does in place what
`ProbabilityField.update(indices, weights)` does to its two leaf tensors; `prune_probability_field` and
`subdivide_probability_field` return the four leaf tensors that `prune(threshold)` / `subdivide(threshold)` assign
to the module's buffers.
"""
from __future__ import annotations

import ctypes as C

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


def _leaf_tensors(leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores):
    n = leaf_weights.numel()
    if leaf_centers.dtype != torch.float32 or leaf_weights.dtype != torch.float32 or \
            leaf_subdivision_scores.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if leaf_levels.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int")
    if leaf_centers.shape != (n, 3) or leaf_levels.shape != (n,) or leaf_subdivision_scores.shape != (n,) or \
            leaf_weights.dim() != 1:
        raise RuntimeError("leaf tensors of one octree expected: centers (n, 3), levels, weights, scores (n,)")
    tensors = [t.contiguous() for t in (leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores)]
    if not all(t.is_cuda for t in tensors):
        raise RuntimeError("expected tensors on the GPU")
    return tensors, n


def _host_size(initial_cell_size):
    size = torch.as_tensor(initial_cell_size, dtype=torch.float32).flatten().cpu()
    if size.numel() == 1:
        size = size.repeat(3)
    if size.numel() != 3:
        raise RuntimeError("initial_cell_size: one value or one per axis expected")
    return (C.c_float * 3)(*[float(v) for v in size])


def _select_workspace(n, device):
    ws_bytes = int(_lib.lib().inpc_field_select_workspace_bytes(n))
    return torch.empty(ws_bytes, dtype=torch.uint8, device=device), ws_bytes


@torch.no_grad()
def prune_probability_field(leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores, threshold: float):
    """The leaves with weight > threshold, in order: (centers, levels, weights, scores), as
    ProbabilityField.prune assigns them (Modules/ProbabilityField.py:159-165). Reads the count back, like the
    reference's boolean indexing."""
    (centers, levels, weights, scores), n = _leaf_tensors(leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores)
    device = weights.device
    out = (torch.empty((n, 3), dtype=torch.float32, device=device), torch.empty(n, dtype=torch.int32, device=device),
           torch.empty(n, dtype=torch.float32, device=device), torch.empty(n, dtype=torch.float32, device=device))
    count = torch.zeros(1, dtype=torch.int32, device=device)
    ws, ws_bytes = _select_workspace(n, device)
    _lib.check(_lib.lib().inpc_field_prune(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(scores), n,
                                           float(threshold), *(_lib.ptr(t) for t in out), _lib.ptr(count), _lib.ptr(ws),
                                           ws_bytes, _lib.current_stream()), "inpc_field_prune")
    kept = int(count.item())
    return tuple(t[:kept].contiguous() for t in out)


@torch.no_grad()
def subdivide_probability_field(leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores, initial_cell_size,
                                threshold: float, max_level: int = 6, max_leaves: int = 16_777_216):
    """The leaf tensors after splitting every leaf with score > threshold and level < max_level into eight, as
    ProbabilityField.subdivide assigns them (Modules/ProbabilityField.py:217-257): (centers, levels, weights,
    scores), or None when the octree would exceed max_leaves (the reference returns without a change, :223-224)."""
    (centers, levels, weights, scores), n = _leaf_tensors(leaf_centers, leaf_levels, leaf_weights, leaf_subdivision_scores)
    device = weights.device
    lib = _lib.lib()
    size_host = _host_size(initial_cell_size)
    count = torch.zeros(1, dtype=torch.int32, device=device)
    ws, ws_bytes = _select_workspace(n, device)
    stream = _lib.current_stream()
    _lib.check(lib.inpc_field_select_count(_lib.ptr(scores), _lib.ptr(levels), n, float(threshold), int(max_level),
                                           _lib.ptr(count), _lib.ptr(ws), ws_bytes, stream), "inpc_field_select_count")
    n_split = int(count.item())
    if n_split * 8 + (n - n_split) > max_leaves:
        return None
    total = n + 7 * n_split
    out = (torch.empty((total, 3), dtype=torch.float32, device=device), torch.empty(total, dtype=torch.int32, device=device),
           torch.empty(total, dtype=torch.float32, device=device), torch.empty(total, dtype=torch.float32, device=device))
    _lib.check(lib.inpc_field_subdivide(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(scores), n,
                                        float(threshold), int(max_level), size_host, *(_lib.ptr(t) for t in out),
                                        _lib.ptr(count), _lib.ptr(ws), ws_bytes, stream), "inpc_field_subdivide")
    return out


@torch.no_grad()
def morton_encode(positions: torch.Tensor) -> torch.Tensor:
    """(n,) int64 Morton codes of (n, 3) float positions in their bounding cube, 21 bits per axis, x in the lowest
    bit: the role of `CudaUtils.MortonEncoding.morton_encode` in Modules/ProbabilityField.py:142 (that extension's
    source is not part of the reference tree; this is the textbook Z-order code)."""
    if positions.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if positions.dim() != 2 or positions.shape[1] != 3:
        raise RuntimeError("positions (n, 3) expected")
    if not positions.is_cuda:
        raise RuntimeError("expected tensors on the GPU")
    positions = positions.contiguous()
    n = positions.shape[0]
    if n >= 2 ** 32:
        raise RuntimeError("too many positions")
    codes = torch.empty(n, dtype=torch.int64, device=positions.device)
    lib = _lib.lib()
    ws_bytes = int(lib.inpc_morton_workspace_bytes())
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=positions.device)
    _lib.check(lib.inpc_morton_encode(_lib.ptr(positions), n, _lib.ptr(codes), _lib.ptr(ws), ws_bytes,
                                      _lib.current_stream()), "inpc_morton_encode")
    return codes


@torch.no_grad()
def extract_global_samples(leaf_centers: torch.Tensor, leaf_levels: torch.Tensor, initial_cell_size,
                           counts: torch.Tensor, use_morton_order: bool = False) -> torch.Tensor:
    """Quasi-random positions, counts[l] of them in leaf l, leaves in order: what ProbabilityField.extract_global
    computes behind its multinomial draw (Modules/ProbabilityField.py:131-143; Halton points in the cell, the centre
    for a leaf with a single sample; with `use_morton_order` sorted by `morton_encode`). `counts` is the result of
    `torch.bincount(indices, minlength=n_leaves)`."""
    if leaf_centers.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    if leaf_levels.dtype != torch.int32:
        raise RuntimeError("expected scalar type Int")
    if counts.dtype != torch.int64:
        raise RuntimeError("expected scalar type Long")
    n = leaf_levels.numel()
    if leaf_centers.shape != (n, 3) or counts.shape != (n,):
        raise RuntimeError("centers (n, 3), levels (n,) and counts (n,) of one octree expected")
    centers, levels, counts = leaf_centers.contiguous(), leaf_levels.contiguous(), counts.contiguous()
    if not (centers.is_cuda and levels.is_cuda and counts.is_cuda):
        raise RuntimeError("expected tensors on the GPU")
    n_samples = int(counts.sum().item())   # the reference reads it as well (utils.py:58)
    device = centers.device
    positions = torch.empty((n_samples, 3), dtype=torch.float32, device=device)
    lib = _lib.lib()
    ws_bytes = int(lib.inpc_extract_global_workspace_bytes(n))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
    stream = _lib.current_stream()
    _lib.check(lib.inpc_extract_global(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(counts), n,
                                       _host_size(initial_cell_size), _lib.ptr(positions), n_samples, _lib.ptr(ws),
                                       ws_bytes, stream), "inpc_extract_global")
    _lib.check(lib.inpc_extract_global_check(_lib.ptr(ws), n_samples, stream), "inpc_extract_global")
    if use_morton_order:
        positions = positions[torch.argsort(morton_encode(positions))].contiguous()
    return positions
