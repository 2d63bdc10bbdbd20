"""inpc_amd — MI355X (gfx950) implementation of the INPCCudaBackend hot path.

Re-exports the operator API of the reference's INPCCudaBackend package
(INPCCudaBackend/__init__.py:14-22) for the parts this library covers: the octree point sampler and
the bilinear point rasterizer. Native code lives in libinpc_hip.so (build: python -m inpc_amd.build).
"""
from .field import update_probability_field
from .misc import feature_to_opacity, spherical_contraction
from .rasterization import INPCRasterizer, RasterizerMode, RasterizerSettings, rasterize_points
from .sampling import ProbabilityFieldSampler, compute_viewpoint_weights
from .views import PerspectiveCamera, View

__all__ = [
    "INPCRasterizer", "RasterizerSettings", "RasterizerMode", "rasterize_points",
    "ProbabilityFieldSampler", "compute_viewpoint_weights", "update_probability_field",
    "spherical_contraction", "feature_to_opacity",
    "PerspectiveCamera", "View",
]
