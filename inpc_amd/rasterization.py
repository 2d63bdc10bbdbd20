"""Rasterizer operator API: `INPCRasterizer`, `RasterizerSettings`, `RasterizerMode`.

Same names, arguments and error behaviour as B/torch_bindings/rasterization.py:15-189; the native
side is libinpc_hip.so instead of the pybind11 module `_C`. On top of the reference's fixed shape
(8x8 tiles, (N,36) fp16 SH features -> 4 channels) the constructor accepts a tile size, and
`rasterize_points` exposes the direct-feature variants (C in {4, 8, 16}, fp32 or fp16 storage).

Both footprints of the reference are there: BILINEAR (2x2 splat) and GAUSSIAN (screen-space Gaussian,
B/rasterization/src/gaussian/). A Gaussian point touches any number of tiles, so that mode reads the
instance count back after the forward pass, as the reference does, and repeats the pass with larger
buffers in the rare case that they were too small.
"""
from __future__ import annotations

import ctypes as C
import logging
from enum import Enum
from typing import Any, NamedTuple, Optional

import torch
from torch.autograd.function import once_differentiable

from . import _lib
from .views import is_perspective

_log = logging.getLogger("inpc_amd")


class RasterizerMode(Enum):
    BILINEAR = 0
    GAUSSIAN = 1


class RasterizerSettings(NamedTuple):
    w2c: torch.Tensor
    cam_position: torch.Tensor
    mode: RasterizerMode
    width: int
    height: int
    focal_x: float
    focal_y: float
    center_x: float
    center_y: float
    near_plane: float
    far_plane: float

    def as_tuple(self) -> tuple:
        return (self.w2c, self.cam_position, self.mode.value, self.width, self.height, self.focal_x, self.focal_y,
                self.center_x, self.center_y, self.near_plane, self.far_plane)

    def camera(self) -> _lib.Camera:
        return _lib.Camera(int(self.width), int(self.height), float(self.focal_x), float(self.focal_y),
                           float(self.center_x), float(self.center_y), float(self.near_plane), float(self.far_plane))


_FEATURE_MODES = {"sh36": _lib.FEAT_SH36_F16, "f32": _lib.FEAT_DIRECT_F32, "f16": _lib.FEAT_DIRECT_F16,
                  "raw37": _lib.FEAT_RAW37_F16}


def _require_known_mode(settings: RasterizerSettings) -> None:
    if settings.mode not in (RasterizerMode.BILINEAR, RasterizerMode.GAUSSIAN):
        # std::runtime_error("unsupported rasterizer mode"), B/rasterization/src/rasterization_api.cu:102-103
        raise RuntimeError("unsupported rasterizer mode")


# instances per point the Gaussian buffers are sized for beyond the default, learnt from earlier calls
_gaussian_capacity_hint = {"per_point": 0.0}


def _config(settings: RasterizerSettings, n_points: int, tile: int, channels: int, feature_mode: int,
            inference: bool, max_instances: int = 0) -> _lib.RasterConfig:
    return _lib.RasterConfig(int(n_points), int(tile), int(channels), int(feature_mode),
                             _lib.RASTER_INFERENCE if inference else 0, settings.camera(), int(max_instances))


# The bilinear workspace is sized for four instances per point, which no input can exceed, so that no count has to
# come back to the host after the forward pass (the reference reads its instance count back on every call to size
# its buffers, B/rasterization/src/bilinear/forward.cu:86-89): up to this many points and this many bytes (4.5 GB for
# 8,388,608 points with a backward pass: room is not what a 288 GB device lacks, and memory that holds no instance
# is never touched). Beyond either limit the library's default capacity (what evenly spread points need, with a
# margin) is used, the counters are read back, and the call is repeated with room for everything if they say so.
_ALWAYS_FITS_POINTS = 1 << 26
_ALWAYS_FITS_BYTES = 48 << 30


def query_layout(cfg: _lib.RasterConfig) -> _lib.RasterLayout:
    layout = _lib.RasterLayout()
    _lib.check(_lib.lib().inpc_raster_layout_query(C.byref(cfg), C.byref(layout)), "inpc_raster_layout_query")
    return layout


def _checked_inputs(positions, features, opacities, feature_mode: int, channels: int):
    positions = positions.contiguous()
    features = features.contiguous()
    if positions.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float")
    want = torch.float32 if feature_mode == _lib.FEAT_DIRECT_F32 else torch.float16
    if features.dtype != want:
        raise RuntimeError("expected scalar type Float" if want == torch.float32 else "expected scalar type Half")
    n = positions.shape[0]
    width = {_lib.FEAT_SH36_F16: 36, _lib.FEAT_RAW37_F16: 37}.get(feature_mode, channels)
    if features.numel() != n * width:
        raise RuntimeError(f"features must hold {width} values per point")
    if opacities is not None:
        opacities = opacities.contiguous()
        if opacities.dtype != torch.float32:
            raise RuntimeError("expected scalar type Float")
        if opacities.numel() != n:
            raise RuntimeError("opacities must hold one value per point")
    if not positions.is_cuda or not features.is_cuda or (opacities is not None and not opacities.is_cuda):
        raise RuntimeError("expected tensors on the GPU")
    if features.device != positions.device or (opacities is not None and opacities.device != positions.device):
        raise RuntimeError("expected all tensors on the same device")
    return positions, features, opacities


def _new_workspace(n_bytes: int, device) -> torch.Tensor:
    """Uninitialised device bytes for one forward pass (the device allocator aligns them to 256 bytes and more)."""
    return torch.empty(n_bytes, dtype=torch.uint8, device=device)


def _checked_camera_tensor(t: torch.Tensor, numel: int, name: str, device) -> torch.Tensor:
    """The camera tensors reach the kernels as raw float pointers: they must be fp32 on the points' device
    (the reference's data_ptr<float>() raises for another dtype, B/rasterization/src/rasterization_api.cu:61-65)."""
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a tensor")
    if t.dtype != torch.float32:
        raise RuntimeError(f"expected scalar type Float for {name}")
    if t.device != device:
        raise RuntimeError(f"expected {name} on the device of the points ({device})")
    if t.numel() != numel:
        raise RuntimeError(f"{name} must hold {numel} values")
    return t.contiguous()


def _forward_gaussian(settings: RasterizerSettings, positions, features, opacities, tile: int, channels: int,
                      feature_mode: int, inference: bool, scales, sigma_world: float, sigma_cutoff: float):
    """Runs inpc_gaussian_forward; same return value as _forward_native, cfg is a GaussianConfig."""
    n = positions.shape[0]
    device = positions.device
    sh = feature_mode in (_lib.FEAT_SH36_F16, _lib.FEAT_RAW37_F16)
    out_channels = 4 if sh else channels
    H, W = settings.height, settings.width
    image = torch.empty((out_channels, H, W), dtype=torch.float32, device=device)
    alpha = torch.empty((1, H, W), dtype=torch.float32, device=device)
    weights = None if inference else torch.empty(n, dtype=torch.float32, device=device)
    depth = torch.empty((1, H, W), dtype=torch.float32, device=device) if inference else None
    w2c = _checked_camera_tensor(settings.w2c, 16, "w2c", device)
    cam_position = _checked_camera_tensor(settings.cam_position, 3, "cam_position", device)
    if scales is not None:
        scales = scales.contiguous()
        if scales.dtype != torch.float32:
            raise RuntimeError("expected scalar type Float")
        if not scales.is_cuda or scales.device != device:
            raise RuntimeError("expected scales on the device of the points")
        if scales.numel() != n:
            raise RuntimeError("scales must hold one value per point")
    capacity = int(4 * n + 65536 + _gaussian_capacity_hint["per_point"] * n)
    lib = _lib.lib()
    for _ in range(3):
        capacity = min(capacity, 2**31 - 1)
        cfg = _lib.GaussianConfig(_config(settings, n, tile, out_channels, feature_mode, inference),
                                  float(sigma_world), float(sigma_cutoff), capacity, 0)
        layout = _lib.GaussianLayout()
        _lib.check(lib.inpc_gaussian_layout_query(C.byref(cfg), C.byref(layout)), "inpc_gaussian_layout_query")
        workspace = _new_workspace(layout.total_bytes, device)
        stream = _lib.current_stream()
        _lib.check(lib.inpc_gaussian_forward(C.byref(cfg), _lib.ptr(positions), _lib.ptr(features), _lib.ptr(opacities),
                                             _lib.ptr(scales), _lib.ptr(w2c), _lib.ptr(cam_position), _lib.ptr(image),
                                             _lib.ptr(alpha), _lib.ptr(weights), _lib.ptr(depth), _lib.ptr(workspace),
                                             layout.total_bytes, stream), "inpc_gaussian_forward")
        counters = (C.c_uint32 * 4)()
        rc = lib.inpc_gaussian_read_counters(C.byref(cfg), _lib.ptr(workspace), C.byref(counters), stream)
        if rc == 0:
            return image, alpha, (depth if inference else weights), workspace, cfg
        if counters[1] <= capacity:
            _lib.check(rc, "inpc_gaussian_read_counters")
        # the instances did not fit: remember the density and go again with room for all of them
        _gaussian_capacity_hint["per_point"] = max(_gaussian_capacity_hint["per_point"], 1.25 * counters[1] / max(n, 1))
        if counters[1] >= 2**32 - 1:
            break
        capacity = int(counters[1]) + 65536
        del workspace
    raise _lib.BackendError("the points touch more tiles than the instance buffers can index (2^31)")


def _forward_native(settings: RasterizerSettings, positions, features, opacities, tile: int, channels: int,
                    feature_mode: int, inference: bool, scales=None, sigma_world: float = 0.0,
                    sigma_cutoff: float = 3.0):
    """Runs inpc_raster_forward (or inpc_gaussian_forward). Returns (image, alpha, third, workspace, cfg) where
    `third` is the blending weights (training) or the depth image (inference)."""
    _require_known_mode(settings)
    if settings.mode == RasterizerMode.GAUSSIAN:
        return _forward_gaussian(settings, positions, features, opacities, tile, channels, feature_mode, inference,
                                 scales, sigma_world, sigma_cutoff)
    n = positions.shape[0]
    device = positions.device
    sh = feature_mode in (_lib.FEAT_SH36_F16, _lib.FEAT_RAW37_F16)
    out_channels = 4 if sh else channels
    H, W = settings.height, settings.width
    image = torch.empty((out_channels, H, W), dtype=torch.float32, device=device)
    alpha = torch.empty((1, H, W), dtype=torch.float32, device=device)
    weights = None if inference else torch.empty(n, dtype=torch.float32, device=device)
    depth = torch.empty((1, H, W), dtype=torch.float32, device=device) if inference else None
    w2c = _checked_camera_tensor(settings.w2c, 16, "w2c", device)
    cam_position = _checked_camera_tensor(settings.cam_position, 3, "cam_position", device)
    lib = _lib.lib()
    everything = max(4 * n, 1)
    capacity = everything if n <= _ALWAYS_FITS_POINTS else 0
    if capacity and query_layout(_config(settings, n, tile, out_channels, feature_mode, inference,
                                         capacity)).total_bytes > _ALWAYS_FITS_BYTES:
        capacity = 0
    for _ in range(2):
        cfg = _config(settings, n, tile, out_channels, feature_mode, inference, capacity)
        layout = query_layout(cfg)
        workspace = _new_workspace(layout.total_bytes, device)
        stream = _lib.current_stream()
        _lib.check(lib.inpc_raster_forward(C.byref(cfg), _lib.ptr(positions), _lib.ptr(features), _lib.ptr(opacities),
                                           _lib.ptr(w2c), _lib.ptr(cam_position), _lib.ptr(image), _lib.ptr(alpha),
                                           _lib.ptr(weights), _lib.ptr(depth), _lib.ptr(workspace), layout.total_bytes,
                                           stream), "inpc_raster_forward")
        if layout.max_instances >= everything:
            break
        counters = (C.c_uint32 * 3)()
        rc = lib.inpc_raster_read_counters(C.byref(cfg), _lib.ptr(workspace), C.byref(counters), stream)
        if rc == 0:
            break
        if rc != _lib.E_WORKSPACE:
            _lib.check(rc, "inpc_raster_read_counters")
        # the points touch more tiles than the default capacity holds: once more with room for all of them
        capacity = everything
        del workspace
    return image, alpha, (depth if inference else weights), workspace, cfg


class _Rasterize(torch.autograd.Function):
    """Counterpart of B/torch_bindings/rasterization.py:49-101."""

    @staticmethod
    def forward(ctx: Any, positions: torch.Tensor, features: torch.Tensor, opacities: torch.Tensor,
                rasterizer_settings: RasterizerSettings, tile: int = 8, feature_mode: int = _lib.FEAT_SH36_F16,
                channels: int = 4):
        _require_known_mode(rasterizer_settings)
        positions, features, opacities = _checked_inputs(positions, features, opacities, feature_mode, channels)
        image, alpha, blending_weights, workspace, cfg = _forward_native(
            rasterizer_settings, positions, features, opacities, tile, channels, feature_mode, inference=False)
        ctx.save_for_backward(image, alpha, positions, workspace)
        ctx.features_shape, ctx.opacities_shape = features.shape, opacities.shape
        ctx.rasterizer_settings = rasterizer_settings
        ctx.cfg = cfg
        ctx.mark_non_differentiable(blending_weights)
        ctx.set_materialize_grads(False)
        return image, alpha, blending_weights

    @staticmethod
    @once_differentiable
    def backward(ctx: Any, grad_image: Optional[torch.Tensor], grad_alpha: Optional[torch.Tensor], _):
        image, alpha, positions, workspace = ctx.saved_tensors
        cfg = ctx.cfg
        gaussian = isinstance(cfg, _lib.GaussianConfig)
        base = cfg.base if gaussian else cfg
        settings = ctx.rasterizer_settings
        n = positions.shape[0]
        device = positions.device
        # set_materialize_grads(False): an output nobody used arrives as None; substitute zeros
        grad_image = torch.zeros_like(image) if grad_image is None else grad_image.contiguous()
        grad_alpha = torch.zeros_like(alpha) if grad_alpha is None else grad_alpha.contiguous()
        if grad_image.dtype != torch.float32 or grad_alpha.dtype != torch.float32:
            raise RuntimeError("expected scalar type Float")
        if grad_image.device != device or grad_alpha.device != device:
            raise RuntimeError("expected the gradients on the device of the points")
        if grad_image.shape != image.shape or grad_alpha.shape != alpha.shape:
            raise RuntimeError("gradient shapes differ from the outputs")
        mode = base.feature_mode
        scratch = None
        if mode == _lib.FEAT_SH36_F16:
            grad_features = torch.empty((n, 36), dtype=torch.float16, device=device)
            scratch = torch.empty((n, 4), dtype=torch.float32, device=device)
        elif mode == _lib.FEAT_DIRECT_F16:
            grad_features = torch.empty((n, base.channels), dtype=torch.float16, device=device)
            scratch = torch.empty((n, base.channels), dtype=torch.float32, device=device)
        else:
            grad_features = torch.empty((n, base.channels), dtype=torch.float32, device=device)
        grad_opacities = torch.empty((n, 1), dtype=torch.float32, device=device)
        cam_position = _checked_camera_tensor(settings.cam_position, 3, "cam_position", device)
        backward = _lib.lib().inpc_gaussian_backward if gaussian else _lib.lib().inpc_raster_backward
        _lib.check(backward(C.byref(cfg), _lib.ptr(grad_image), _lib.ptr(grad_alpha), _lib.ptr(image), _lib.ptr(alpha),
                            _lib.ptr(positions), _lib.ptr(cam_position), _lib.ptr(grad_features),
                            _lib.ptr(grad_opacities), _lib.ptr(scratch), _lib.ptr(workspace), workspace.numel(),
                            _lib.current_stream()),
                   "inpc_gaussian_backward" if gaussian else "inpc_raster_backward")
        grad_features = grad_features.view(ctx.features_shape)
        grad_opacities = grad_opacities.view(ctx.opacities_shape)
        return None, grad_features, grad_opacities, None, None, None, None


class INPCRasterizer(torch.nn.Module):
    """Counterpart of B/torch_bindings/rasterization.py:104-189. The reference's tiles are 8x8
    (B/rasterization/include/bilinear/config.h:23-25, gaussian/config.h:23-25). `tile` = 8 or 16 fixes the size;
    left at None, every mode gets the size that is fastest here without changing its results: 16 for the bilinear
    footprint (its image does not depend on the tile size: a point reaches the same pixels either way), 8 for the
    Gaussian one (whose tile bounds decide which pixels at the rim of a footprint are drawn)."""

    def __init__(self, tile: Optional[int] = None) -> None:
        super().__init__()
        if tile not in (None, 8, 16):
            raise ValueError("tile must be 8 or 16")
        self.tile = tile

    def tile_for(self, mode: RasterizerMode) -> int:
        if self.tile is not None:
            return self.tile
        return 8 if mode == RasterizerMode.GAUSSIAN else 16

    @staticmethod
    def extract_settings(view, mode: int) -> RasterizerSettings:
        if not is_perspective(view.camera):
            raise NotImplementedError
        if getattr(view.camera, "distortion", None) is not None:
            _log.warning("rasterizer ignores all distortion parameters")
        try:
            rasterizer_mode = RasterizerMode(mode)
        except ValueError:
            _log.warning("invalid rasterizer mode %s, defaulting to BILINEAR", mode)
            rasterizer_mode = RasterizerMode.BILINEAR
        return RasterizerSettings(view.w2c, view.position, rasterizer_mode, view.camera.width, view.camera.height,
                                  view.camera.focal_x, view.camera.focal_y, view.camera.center_x,
                                  view.camera.center_y, view.camera.near_plane, view.camera.far_plane)

    @staticmethod
    def extract_base_sigma_world(camera) -> float:
        if not is_perspective(camera):
            raise NotImplementedError
        return 0.05 / camera.focal_y

    def forward(self, view, mode: int, positions: torch.Tensor, features: torch.Tensor,
                opacities: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(image (4,H,W), alpha (1,H,W), blending_weights (N,)); differentiable in features and
        opacities, positions get no gradient."""
        settings = self.extract_settings(view, mode)
        return _Rasterize.apply(positions, features, opacities, settings, self.tile_for(settings.mode),
                                _lib.FEAT_SH36_F16, 4)

    def render(self, view, mode: int, positions: torch.Tensor, features_raw: torch.Tensor,
               sigma_world_scale: float, sigma_cutoff: float) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """(image, depth, alpha) from raw (N,37) fp16 appearance output; the sigma arguments only
        concern the Gaussian footprint and are ignored by the bilinear one, as in the reference."""
        settings = self.extract_settings(view, mode)
        _require_known_mode(settings)
        positions, features_raw, _ = _checked_inputs(positions, features_raw, None, _lib.FEAT_RAW37_F16, 4)
        sigma_world = sigma_world_scale * self.extract_base_sigma_world(view.camera)
        image, alpha, depth, _, _ = _forward_native(settings, positions, features_raw, None, self.tile_for(settings.mode), 4,
                                                    _lib.FEAT_RAW37_F16, inference=True, sigma_world=sigma_world,
                                                    sigma_cutoff=sigma_cutoff)
        return image, depth, alpha

    def render_preextracted(self, view, mode: int, positions: torch.Tensor, features: torch.Tensor,
                            opacities: torch.Tensor, scales: Optional[torch.Tensor] = None,
                            sigma_world_scale: float = 1.0,
                            sigma_cutoff: float = 3.0) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        settings = self.extract_settings(view, mode)
        _require_known_mode(settings)
        positions, features, opacities = _checked_inputs(positions, features, opacities, _lib.FEAT_SH36_F16, 4)
        if scales is not None and scales.numel() == 0:   # the reference passes an empty tensor for "no scales"
            scales = None
        sigma_world = sigma_world_scale * self.extract_base_sigma_world(view.camera)
        image, alpha, depth, _, _ = _forward_native(settings, positions, features, opacities, self.tile_for(settings.mode), 4,
                                                    _lib.FEAT_SH36_F16, inference=True, scales=scales,
                                                    sigma_world=sigma_world, sigma_cutoff=sigma_cutoff)
        return image, depth, alpha


def rasterize_points(view, positions: torch.Tensor, features: torch.Tensor, opacities: torch.Tensor, tile: int = 16,
                     inference: bool = False, mode: int = RasterizerMode.BILINEAR.value,
                     scales: Optional[torch.Tensor] = None, sigma_world: float = 0.0, sigma_cutoff: float = 3.0):
    """Direct-feature rasterization: features (N,C), C in {4, 8, 16}, fp32 or fp16 storage, blended as
    they are. Training: (image (C,H,W), alpha, blending_weights), differentiable in features and
    opacities. Inference: (image, depth, alpha); scales, sigma_world and sigma_cutoff concern the Gaussian
    footprint's inference variant only."""
    settings = INPCRasterizer.extract_settings(view, mode)
    channels = features.shape[-1]
    if features.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("expected scalar type Float or Half")
    feature_mode = _lib.FEAT_DIRECT_F32 if features.dtype == torch.float32 else _lib.FEAT_DIRECT_F16
    if inference:
        positions, features, opacities = _checked_inputs(positions, features, opacities, feature_mode, channels)
        image, alpha, depth, _, _ = _forward_native(settings, positions, features, opacities, tile, channels,
                                                    feature_mode, inference=True, scales=scales,
                                                    sigma_world=sigma_world, sigma_cutoff=sigma_cutoff)
        return image, depth, alpha
    return _Rasterize.apply(positions, features, opacities, settings, tile, feature_mode, channels)
