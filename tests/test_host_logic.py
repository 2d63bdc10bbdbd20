"""Host-side mirror of the reference's operator interface: settings extraction, mode handling, argument errors
(B/torch_bindings/rasterization.py:104-189, B/torch_bindings/sampling.py:9-132). CPU only: every case here ends
in Python before a kernel would be launched."""
import logging

import numpy as np
import pytest
import torch

import inpc_amd
from inpc_amd import _lib, synthetic
from inpc_amd.rasterization import INPCRasterizer, RasterizerMode, RasterizerSettings, rasterize_points
from inpc_amd.sampling import ProbabilityFieldSampler, compute_viewpoint_weights
from inpc_amd.views import PerspectiveCamera, View, is_perspective


class Orthographic:
    width, height = 10, 10


def cpu_view(camera=None):
    camera = camera or PerspectiveCamera(64, 48, 50.0, 51.0, 32.5, 24.25, 0.1, 10.0)
    return View(camera, torch.eye(4), torch.zeros(3))


def test_public_names_match_the_reference_package():
    for name in ("INPCRasterizer", "RasterizerSettings", "RasterizerMode", "ProbabilityFieldSampler",
                 "compute_viewpoint_weights"):
        assert hasattr(inpc_amd, name)
    assert [m.name for m in RasterizerMode] == ["BILINEAR", "GAUSSIAN"] and RasterizerMode.BILINEAR.value == 0


def test_extract_settings_unpacks_the_view_in_reference_order():
    view = cpu_view()
    s = INPCRasterizer.extract_settings(view, 0)
    assert isinstance(s, RasterizerSettings) and s.mode is RasterizerMode.BILINEAR
    t = s.as_tuple()
    assert t[0] is view.w2c and t[1] is view.position
    assert t[2:] == (0, 64, 48, 50.0, 51.0, 32.5, 24.25, 0.1, 10.0)
    cam = s.camera()
    assert (cam.width, cam.height) == (64, 48) and cam.center_y == 24.25 and cam.near_plane == np.float32(0.1)


def test_invalid_mode_defaults_to_bilinear_with_a_warning(caplog):
    with caplog.at_level(logging.WARNING, logger="inpc_amd"):
        s = INPCRasterizer.extract_settings(cpu_view(), 7)
    assert s.mode is RasterizerMode.BILINEAR and "invalid rasterizer mode" in caplog.text


def test_distortion_is_ignored_by_the_rasterizer_and_refused_by_the_sampler(caplog):
    camera = PerspectiveCamera(64, 48, 50.0, 50.0, 32.0, 24.0, distortion=object())
    with caplog.at_level(logging.WARNING, logger="inpc_amd"):
        INPCRasterizer.extract_settings(cpu_view(camera), 0)
    assert "distortion" in caplog.text
    z = torch.zeros
    with pytest.raises(NotImplementedError):
        compute_viewpoint_weights(z(1, 3), z(1, dtype=torch.int32), z(1), cpu_view(camera), 1.0)
    with pytest.raises(NotImplementedError):
        ProbabilityFieldSampler(1).generate_samples(z(1, 3), z(1, dtype=torch.int32), z(1), cpu_view(camera), 4, 1.0)


def test_non_perspective_cameras_are_not_implemented():
    assert is_perspective(PerspectiveCamera(1, 1, 1.0, 1.0, 0.5, 0.5)) and not is_perspective(Orthographic())
    view = cpu_view(Orthographic())
    with pytest.raises(NotImplementedError):
        INPCRasterizer.extract_settings(view, 0)
    with pytest.raises(NotImplementedError):
        INPCRasterizer.extract_base_sigma_world(Orthographic())
    z = torch.zeros
    with pytest.raises(NotImplementedError):
        compute_viewpoint_weights(z(1, 3), z(1, dtype=torch.int32), z(1), view, 1.0)
    sampler = ProbabilityFieldSampler(0)
    for call in (lambda: sampler.generate_training_samples(z(1, 3), z(1, dtype=torch.int32), z(1), view, 4, 1.0),
                 lambda: sampler.generate_samples(z(1, 3), z(1, dtype=torch.int32), z(1), view, 4, 1.0),
                 lambda: sampler.generate_expected_samples(z(1, 3), z(1, dtype=torch.int32), z(1), view, 4, 2, 1.0)):
        with pytest.raises(NotImplementedError):
            call()


def test_base_sigma_world():
    assert INPCRasterizer.extract_base_sigma_world(PerspectiveCamera(8, 8, 100.0, 200.0, 4, 4)) == 0.05 / 200.0


def test_gaussian_mode_is_a_known_mode():
    # both footprints get as far as the device check (B/torch_bindings/rasterization.py:15-18)
    r = INPCRasterizer()
    n = 4
    args = (torch.zeros(n, 3), torch.zeros(n, 36, dtype=torch.float16), torch.zeros(n))
    for mode in (RasterizerMode.BILINEAR.value, RasterizerMode.GAUSSIAN.value):
        with pytest.raises(RuntimeError, match="expected tensors on the GPU"):
            r(cpu_view(), mode, *args)


def test_tile_argument():
    assert INPCRasterizer(8).tile == 8 and INPCRasterizer(16).tile == 16
    # left open, the tile size follows the mode: the bilinear image does not depend on it, the Gaussian one keeps the
    # reference's 8x8
    auto = INPCRasterizer()
    assert auto.tile_for(RasterizerMode.BILINEAR) == 16 and auto.tile_for(RasterizerMode.GAUSSIAN) == 8
    assert INPCRasterizer(8).tile_for(RasterizerMode.BILINEAR) == 8
    with pytest.raises(ValueError):
        INPCRasterizer(32)


@pytest.mark.parametrize("positions,features,opacities,message", [
    (torch.zeros(4, 3, dtype=torch.float64), torch.zeros(4, 36, dtype=torch.float16), torch.zeros(4), "Float"),
    (torch.zeros(4, 3), torch.zeros(4, 36), torch.zeros(4), "Half"),
    (torch.zeros(4, 3), torch.zeros(4, 35, dtype=torch.float16), torch.zeros(4), "36 values"),
    (torch.zeros(4, 3), torch.zeros(4, 36, dtype=torch.float16), torch.zeros(4, dtype=torch.float16), "Float"),
    (torch.zeros(4, 3), torch.zeros(4, 36, dtype=torch.float16), torch.zeros(3), "one value per point"),
    (torch.zeros(4, 3), torch.zeros(4, 36, dtype=torch.float16), torch.zeros(4), "on the GPU"),
])
def test_rasterizer_argument_errors(positions, features, opacities, message):
    with pytest.raises(RuntimeError, match=message):
        INPCRasterizer()(cpu_view(), 0, positions, features, opacities)
    with pytest.raises(RuntimeError, match=message):
        INPCRasterizer().render_preextracted(cpu_view(), 0, positions, features, opacities)


def test_render_and_direct_feature_argument_errors():
    with pytest.raises(RuntimeError, match="37 values"):
        INPCRasterizer().render(cpu_view(), 0, torch.zeros(4, 3), torch.zeros(4, 36, dtype=torch.float16), 1.0, 3.0)
    with pytest.raises(RuntimeError, match="on the GPU"):
        INPCRasterizer().render(cpu_view(), 0, torch.zeros(4, 3), torch.zeros(4, 37, dtype=torch.float16), 1.0, 3.0)
    with pytest.raises(RuntimeError, match="on the GPU"):
        rasterize_points(cpu_view(), torch.zeros(4, 3), torch.zeros(4, 8), torch.zeros(4))
    with pytest.raises(RuntimeError, match="Float"):
        rasterize_points(cpu_view(), torch.zeros(4, 3), torch.zeros(4, 8, dtype=torch.float64), torch.zeros(4))


def test_sampler_argument_errors():
    view = cpu_view()
    z = torch.zeros
    with pytest.raises(RuntimeError, match="Float"):
        compute_viewpoint_weights(z(2, 3, dtype=torch.float64), z(2, dtype=torch.int32), z(2), view, 1.0)
    with pytest.raises(RuntimeError, match="Int"):
        compute_viewpoint_weights(z(2, 3), z(2, dtype=torch.int64), z(2), view, 1.0)
    with pytest.raises(RuntimeError, match="on the GPU"):
        compute_viewpoint_weights(z(2, 3), z(2, dtype=torch.int32), z(2), view, 1.0)
    with pytest.raises(RuntimeError, match="on the GPU"):
        ProbabilityFieldSampler(3).generate_training_samples(z(2, 3), z(2, dtype=torch.int32), z(2), view, 8, 1.0)


def test_sampler_generator_is_pcg32_seed_stream_1(oracle):
    # B/sampling/include/sampling_api.h:27: the generator is pcg32(seed), i.e. stream 1
    for seed in (0, 42, 2**63 + 5):
        s = ProbabilityFieldSampler(seed)
        ref = oracle.Pcg32(seed, 1)
        assert s.rng_state() == (int(ref.state[0]), int(ref.state[1]))


def test_synthetic_scene_helpers_are_deterministic():
    a = synthetic.octree_leaves(1000, 5)
    b = synthetic.octree_leaves(1000, 5)
    for field in ("centers", "levels", "weights"):
        np.testing.assert_array_equal(getattr(a, field), getattr(b, field))
    assert a.levels.dtype == np.int32 and a.weights.sum() == pytest.approx(1.0, rel=1e-5)
    hv = synthetic.rotated_camera(100, 80, 90.0, 2.0, 0.3, 0.1)
    rot = hv.w2c[:3, :3].astype(np.float64)
    np.testing.assert_allclose(rot @ rot.T, np.eye(3), atol=1e-6)
    # the stored camera position is the point the world-to-camera transform maps to the origin
    np.testing.assert_allclose(rot @ hv.position + hv.w2c[:3, 3], 0, atol=1e-5)


def test_camera_tensors_must_be_fp32_on_the_points_device():
    # w2c and cam_position reach the kernels as raw float pointers: another dtype would be reinterpreted, a host
    # tensor would hand a host address to a kernel. Both are refused before anything is launched.
    from inpc_amd.rasterization import _checked_camera_tensor

    device = torch.device("cuda:0")
    with pytest.raises(RuntimeError, match="Float"):
        _checked_camera_tensor(torch.eye(4, dtype=torch.float64), 16, "w2c", device)
    with pytest.raises(RuntimeError, match="on the device of the points"):
        _checked_camera_tensor(torch.eye(4), 16, "w2c", device)
    with pytest.raises(RuntimeError, match="must hold 3 values"):
        _checked_camera_tensor(torch.zeros(4), 3, "cam_position", torch.device("cpu"))
    with pytest.raises(RuntimeError, match="must be a tensor"):
        _checked_camera_tensor(np.eye(4, dtype=np.float32), 16, "w2c", device)
    ok = _checked_camera_tensor(torch.eye(4).t(), 16, "w2c", torch.device("cpu"))   # made contiguous, otherwise as given
    assert ok.is_contiguous() and ok.dtype == torch.float32


def test_c_module_has_the_eleven_names_with_the_reference_parameter_lists():
    """Names and parameter counts of B/torch_bindings/bindings.cpp:10-29 with rasterization_api.h:8-86,
    sampling_api.h:11-82 and misc_api.h:7-25."""
    import inspect

    from inpc_amd import _C

    expected = {"forward": 14, "backward": 22, "render": 15, "render_preextracted": 17,
                "compute_viewpoint_weights_cuda": 13, "compute_normalized_weight_decay_grads_cuda": 1,
                "add_normalized_weight_decay_grads_cuda": 2, "spherical_contraction_cuda": 1, "cauchy_loss_cuda": 2,
                "cauchy_loss_backward_cuda": 3}
    for name, count in expected.items():
        assert len(inspect.signature(getattr(_C, name)).parameters) == count, name
    sampler = _C.ProbabilityFieldSamplerCUDA
    assert len(inspect.signature(sampler.__init__).parameters) == 2          # self, seed
    assert len(inspect.signature(sampler.generate_training_samples).parameters) == 15
    assert len(inspect.signature(sampler.generate_samples).parameters) == 15
    assert len(inspect.signature(sampler.generate_expected_samples).parameters) == 16
