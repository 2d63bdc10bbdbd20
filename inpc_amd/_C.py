"""The native module's surface: the eleven names of the reference's pybind11 module `INPCCudaBackend._C`
(B/torch_bindings/bindings.cpp:10-29) with the same positional arguments and return values, on top of
libinpc_hip.so. A maintainer who keeps the reference's own `torch_bindings/*.py` only swaps the import
`from INPCCudaBackend import _C` for `from inpc_amd import _C`.

Differences that the reference's Python layer cannot observe:
  * `forward` returns one workspace tensor where the reference returns three buffers (the other two are empty) and
    uses the two integers it hands back (`n_instances`, `instance_primitive_indices_selector`) for its own
    bookkeeping: the capacity of the instance buffers and the tile size. The reference's layer passes all five
    back to `backward` untouched (B/torch_bindings/rasterization.py:57-95).
  * tiles are 16x16 for the bilinear footprint (its results do not depend on the tile size), 8x8 for the Gaussian one.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from . import misc as _misc
from . import rasterization as _raster
from . import sampling as _sampling
from .views import PerspectiveCamera, View


def _settings(w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x, center_y, near_plane,
              far_plane) -> _raster.RasterizerSettings:
    try:
        mode = _raster.RasterizerMode(int(rasterizer_mode))
    except ValueError:
        raise RuntimeError("unsupported rasterizer mode")   # B/rasterization/src/rasterization_api.cu:102-103
    return _raster.RasterizerSettings(w2c, cam_position, mode, int(width), int(height), float(focal_x), float(focal_y),
                                      float(center_x), float(center_y), float(near_plane), float(far_plane))


def _tile(mode: _raster.RasterizerMode) -> int:
    return 8 if mode == _raster.RasterizerMode.GAUSSIAN else 16


# ---- rasterization (B/rasterization/include/rasterization_api.h:8-86) ----------------------------------------
def forward(positions, features, opacities, w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y,
            center_x, center_y, near_plane, far_plane):
    """-> (image (4,H,W), alpha (1,H,W), blending_weights (N,), per_primitive_buffers, per_tile_buffers,
    per_instance_buffers, n_instances, instance_primitive_indices_selector)."""
    settings = _settings(w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x, center_y,
                         near_plane, far_plane)
    positions, features, opacities = _raster._checked_inputs(positions, features, opacities, _lib.FEAT_SH36_F16, 4)
    tile = _tile(settings.mode)
    image, alpha, weights, workspace, cfg = _raster._forward_native(settings, positions, features, opacities, tile, 4,
                                                                    _lib.FEAT_SH36_F16, inference=False)
    capacity = cfg.max_instances   # of the Gaussian or the bilinear configuration: both name the field alike
    empty = torch.empty(0, dtype=torch.uint8, device=positions.device)
    return image, alpha, weights, workspace, empty, empty.clone(), int(capacity), tile


def backward(grad_image, grad_alpha, image, alpha, positions, opacities, per_primitive_buffers, per_tile_buffers,
             per_instance_buffers, w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x,
             center_y, near_plane, far_plane, n_instances, instance_primitive_indices_selector):
    """-> (grad_features (N,36) fp16, grad_opacities (N,1) f32)."""
    settings = _settings(w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x, center_y,
                         near_plane, far_plane)
    positions = positions.contiguous()
    n = positions.shape[0]
    device = positions.device
    tile = int(instance_primitive_indices_selector)
    base = _raster._config(settings, n, tile, 4, _lib.FEAT_SH36_F16, False, int(n_instances))
    gaussian = settings.mode == _raster.RasterizerMode.GAUSSIAN
    cfg = _lib.GaussianConfig(base, 0.0, 3.0, int(n_instances), 0) if gaussian else base
    # an output that nobody used arrives as None (set_materialize_grads(False) in the caller)
    grad_image = torch.zeros_like(image) if grad_image is None else grad_image.contiguous()
    grad_alpha = torch.zeros_like(alpha) if grad_alpha is None else grad_alpha.contiguous()
    if grad_image.shape != image.shape or grad_alpha.shape != alpha.shape:
        raise RuntimeError("gradient shapes differ from the outputs")
    for t in (grad_image, grad_alpha, image, alpha):
        if t.dtype != torch.float32:
            raise RuntimeError("expected scalar type Float")
        if t.device != device:
            raise RuntimeError("expected all tensors on the device of the points")
    workspace = per_primitive_buffers
    grad_features = torch.empty((n, 36), dtype=torch.float16, device=device)
    grad_opacities = torch.empty((n, 1), dtype=torch.float32, device=device)
    scratch = torch.empty((n, 4), dtype=torch.float32, device=device)
    cam_position = _raster._checked_camera_tensor(settings.cam_position, 3, "cam_position", device)
    call = _lib.lib().inpc_gaussian_backward if gaussian else _lib.lib().inpc_raster_backward
    _lib.check(call(C.byref(cfg), _lib.ptr(grad_image), _lib.ptr(grad_alpha), _lib.ptr(image.contiguous()),
                    _lib.ptr(alpha.contiguous()), _lib.ptr(positions), _lib.ptr(cam_position), _lib.ptr(grad_features),
                    _lib.ptr(grad_opacities), _lib.ptr(scratch), _lib.ptr(workspace), workspace.numel(),
                    _lib.current_stream()), "backward")
    return grad_features, grad_opacities


def render(positions, features_raw, w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x,
           center_y, near_plane, far_plane, sigma_world, sigma_cutoff):
    """-> (image (4,H,W), depth (1,H,W), alpha (1,H,W)) from raw (N,37) fp16 appearance output."""
    settings = _settings(w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x, center_y,
                         near_plane, far_plane)
    positions, features_raw, _ = _raster._checked_inputs(positions, features_raw, None, _lib.FEAT_RAW37_F16, 4)
    image, alpha, depth, _, _ = _raster._forward_native(settings, positions, features_raw, None, _tile(settings.mode), 4,
                                                        _lib.FEAT_RAW37_F16, inference=True,
                                                        sigma_world=float(sigma_world), sigma_cutoff=float(sigma_cutoff))
    return image, depth, alpha


def render_preextracted(positions, features, opacities, scales, w2c, cam_position, rasterizer_mode, width, height,
                        focal_x, focal_y, center_x, center_y, near_plane, far_plane, sigma_world, sigma_cutoff):
    """-> (image, depth, alpha); `scales` is an empty tensor for "one size for all points"
    (B/torch_bindings/rasterization.py:176-178)."""
    settings = _settings(w2c, cam_position, rasterizer_mode, width, height, focal_x, focal_y, center_x, center_y,
                         near_plane, far_plane)
    positions, features, opacities = _raster._checked_inputs(positions, features, opacities, _lib.FEAT_SH36_F16, 4)
    if scales is not None and scales.numel() == 0:
        scales = None
    image, alpha, depth, _, _ = _raster._forward_native(settings, positions, features, opacities, _tile(settings.mode), 4,
                                                        _lib.FEAT_SH36_F16, inference=True, scales=scales,
                                                        sigma_world=float(sigma_world), sigma_cutoff=float(sigma_cutoff))
    return image, depth, alpha


# ---- sampling (B/sampling/include/sampling_api.h:11-82) ------------------------------------------------------
def _view(w2c, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane) -> View:
    camera = PerspectiveCamera(int(width), int(height), float(focal_x), float(focal_y), float(center_x), float(center_y),
                               float(near_plane), float(far_plane))
    return View(camera, w2c, None)


def compute_viewpoint_weights_cuda(centers, levels, weights, w2c, width, height, focal_x, focal_y, center_x, center_y,
                                   near_plane, far_plane, initial_size):
    view = _view(w2c, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
    return _sampling.compute_viewpoint_weights(centers, levels, weights, view, float(initial_size))


class ProbabilityFieldSamplerCUDA:
    """Counterpart of sampling_api::ProbabilityFieldSampler: a generator seeded as pcg32(seed) and three draws."""

    def __init__(self, seed: int) -> None:
        self._sampler = _sampling.ProbabilityFieldSampler(int(seed))

    def generate_training_samples(self, centers, levels, weights, w2c, n_samples, width, height, focal_x, focal_y,
                                  center_x, center_y, near_plane, far_plane, initial_size):
        view = _view(w2c, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
        return self._sampler.generate_training_samples(centers, levels, weights, view, int(n_samples),
                                                       float(initial_size))

    def generate_samples(self, centers, levels, weights, w2c, n_samples, width, height, focal_x, focal_y, center_x,
                         center_y, near_plane, far_plane, initial_size):
        view = _view(w2c, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
        return self._sampler.generate_samples(centers, levels, weights, view, int(n_samples), float(initial_size))

    def generate_expected_samples(self, centers, levels, weights, w2c, n_samples, n_multi, width, height, focal_x,
                                  focal_y, center_x, center_y, near_plane, far_plane, initial_size):
        view = _view(w2c, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
        return self._sampler.generate_expected_samples(centers, levels, weights, view, int(n_samples), int(n_multi),
                                                       float(initial_size))


# ---- misc (B/misc/include/misc_api.h:7-25) -------------------------------------------------------------------
def compute_normalized_weight_decay_grads_cuda(weights):
    return _misc.compute_normalized_weight_decay_grads(weights)


def add_normalized_weight_decay_grads_cuda(weights, grads) -> None:
    weights = _misc._require_gpu_float(weights)
    if grads.dtype != torch.float32 or not grads.is_cuda or not grads.is_contiguous():
        raise RuntimeError("expected a contiguous Float tensor on the GPU")
    _lib.check(_lib.lib().inpc_weight_decay_grads(_lib.ptr(weights), _lib.ptr(grads), weights.shape[0], 1,
                                                  _lib.current_stream()), "inpc_weight_decay_grads")


def spherical_contraction_cuda(positions):
    return _misc.spherical_contraction(positions)


def cauchy_loss_cuda(input, target):
    """-> the loss (sum over the element-wise terms, B/misc/src/misc_api.cu:51-65)."""
    input, target = _misc._require_gpu_float(input), _misc._require_gpu_float(target)
    elementwise = torch.empty_like(input)
    _lib.check(_lib.lib().inpc_cauchy_loss(_lib.ptr(input), _lib.ptr(target), _lib.ptr(elementwise), input.numel(),
                                           _lib.current_stream()), "inpc_cauchy_loss")
    return elementwise.sum()


def cauchy_loss_backward_cuda(grad, input, target):
    input, target = _misc._require_gpu_float(input), _misc._require_gpu_float(target)
    grad = _misc._require_gpu_float(grad.reshape(1))
    grad_input = torch.empty_like(input)
    _lib.check(_lib.lib().inpc_cauchy_loss_backward(_lib.ptr(grad), _lib.ptr(input), _lib.ptr(target),
                                                    _lib.ptr(grad_input), input.numel(), _lib.current_stream()),
               "inpc_cauchy_loss_backward")
    return grad_input
