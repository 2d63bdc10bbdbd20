"""inpc_amd — MI355X (gfx950) implementation of the INPCCudaBackend hot path.

Re-exports the operator API of the reference's INPCCudaBackend package
(INPCCudaBackend/__init__.py:14-22) for the parts this library covers: the octree point sampler and
the bilinear point rasterizer. Native code lives in libinpc_hip.so (build: python -m inpc_amd.build).
"""
from .field import extract_global_samples, morton_encode, prune_probability_field, subdivide_probability_field, update_probability_field
from .misc import (add_normalized_weight_decay_grads, compute_normalized_weight_decay_grads, feature_to_opacity,
                   fused_cauchy_loss, spherical_contraction)
from .rasterization import INPCRasterizer, RasterizerMode, RasterizerSettings, rasterize_points
from .sampling import ProbabilityFieldSampler, compute_viewpoint_weights
from .views import PerspectiveCamera, View

__all__ = [
    "INPCRasterizer", "RasterizerSettings", "RasterizerMode", "rasterize_points",
    "ProbabilityFieldSampler", "compute_viewpoint_weights", "update_probability_field", "prune_probability_field", "extract_global_samples", "morton_encode", "subdivide_probability_field",
    "spherical_contraction", "feature_to_opacity", "compute_normalized_weight_decay_grads",
    "add_normalized_weight_decay_grads", "fused_cauchy_loss",
    "PerspectiveCamera", "View",
]
