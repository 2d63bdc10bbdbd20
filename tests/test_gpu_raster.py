"""GPU parity of the rasterizer against the CPU oracle, through the C ABI.

Bit-exact: tile bounds, screen coordinates, depth keys, depth order, instance order, tile ranges.
Within 1e-4 relative (plus a small absolute floor for near-zero values): image, alpha, depth image,
blending weights, feature and opacity gradients.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from inpc_amd import _lib, synthetic
from tests import helpers as H

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def oracle_cfg(O, hv, n, tile, channels, mode, inference=False):
    c = hv.camera
    cam = O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)
    return O.make_config(n, cam, tile, channels, mode, O.RASTER_INFERENCE if inference else 0)


def scene(n, channels, seed=0, width=251, height=163, focal=230.0, side=1.6, distance=2.4, dtype=np.float32):
    hv = synthetic.camera_on_z(width, height, focal, distance)
    pos = synthetic.cube_points(n, side, seed)
    feats, opac = synthetic.point_attributes(n, channels, "normal", seed + 1, dtype)
    return hv, pos, feats, opac


def check_structure(dbg, ref):
    assert dbg["n_visible"] == ref["n_visible"]
    assert dbg["n_instances"] == ref["n_instances"]
    np.testing.assert_array_equal(dbg["n_touched"], ref["n_touched"])
    np.testing.assert_array_equal(dbg["bounds"], ref["bounds"])
    np.testing.assert_array_equal(dbg["screen_xy"].view(np.uint32), ref["screen_xy"].view(np.uint32))
    vis = ref["n_touched"] > 0
    np.testing.assert_array_equal(dbg["depth"][vis].view(np.uint32), ref["depth"][vis].view(np.uint32))
    # the oracle's depth keys are those of its depth-ordered points; here every tile is sorted on its own, so the
    # comparison is per instance, in final (tile, depth bits, point index) order
    key_of_point = np.zeros(len(ref["n_touched"]), np.uint32)
    key_of_point[ref["depth_order"]] = ref["depth_keys"]
    np.testing.assert_array_equal(dbg["instance_keys"], ref["instance_keys"])
    np.testing.assert_array_equal(dbg["instance_points"], ref["instance_points"])
    np.testing.assert_array_equal(dbg["instance_depth_keys"], key_of_point[ref["instance_points"]])
    np.testing.assert_array_equal(dbg["tile_ranges"], ref["tile_ranges"])


@pytest.mark.parametrize("tile", [8, 16])
@pytest.mark.parametrize("channels", [4, 8, 16])
def test_forward_direct_f32(gpu, oracle, tile, channels):
    n = 60000
    hv, pos, feats, opac = scene(n, channels, seed=tile + channels)
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
    ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32), pos, feats, opac,
                                hv.w2c, debug=True)
    dbg = run.debug()
    check_structure(dbg, ref)
    np.testing.assert_array_equal(dbg["features_view"], ref["features_view"])  # copied into the records as they are
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")


@pytest.mark.parametrize("tile", [8, 16])
def test_forward_dense_opaque_scene_terminates_early(gpu, oracle, tile):
    # many points per pixel with high opacity: exercises the transmittance early-out and multi-batch tiles
    n = 200000
    hv = synthetic.camera_on_z(97, 61, 90.0, 2.4)
    pos = synthetic.cube_points(n, 1.2, 5)
    feats, _ = synthetic.point_attributes(n, 4, "uniform", 6)
    opac = np.random.default_rng(7).uniform(0.3, 0.999, n).astype(np.float32)
    run = H.RasterRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_DIRECT_F32).forward()
    ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_DIRECT_F32), pos, feats, opac, hv.w2c,
                                debug=True)
    check_structure(run.debug(), ref)
    out = run.outputs()
    assert (ref["alpha"] == 1.0).mean() > 0.3  # a large share of the pixels saturates
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")


@pytest.mark.parametrize("tile", [8, 16])
def test_forward_sh36_and_backward(gpu, oracle, tile):
    n = 50000
    hv = synthetic.rotated_camera(233, 171, 210.0, 2.6, yaw=0.5, pitch=-0.3)
    pos = synthetic.cube_points(n, 1.5, 11)
    feats = synthetic.sh_features(n, 12)
    _, opac = synthetic.point_attributes(n, 4, "normal", 13)
    run = H.RasterRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_SH36_F16).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_SH36_F16)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, hv.position, debug=True)
    dbg = run.debug()
    check_structure(dbg, ref)
    vis = ref["n_touched"] > 0
    H.assert_close(dbg["features_view"][vis], ref["features_view"][vis], RTOL, 1e-5, "SH view features")
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")

    rng = np.random.default_rng(14)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                               hv.position)
    assert (gf[~vis] == 0).all() and (go[~vis] == 0).all()
    # fp16 outputs: one fp16 ulp of slack on top of the fp32 tolerance
    H.assert_close(gf.astype(np.float32), gf_ref.astype(np.float32), 2e-3, 1e-7, "SH feature gradients")
    H.assert_close(go, go_ref, RTOL, 1e-7, "opacity gradients")


@pytest.mark.parametrize("tile,channels,mode", [(16, 8, "f32"), (8, 4, "f32"), (16, 16, "f32"), (8, 8, "f16"),
                                                (16, 4, "f16")])
def test_backward_direct(gpu, oracle, tile, channels, mode):
    n = 40000
    fmode = _lib.FEAT_DIRECT_F32 if mode == "f32" else _lib.FEAT_DIRECT_F16
    hv, pos, feats, opac = scene(n, channels, seed=31 + channels, dtype=np.float32 if mode == "f32" else np.float16)
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, fmode).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, channels, fmode)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    rng = np.random.default_rng(32)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    # the backward replays against the forward's own outputs, as the autograd function does
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
    if mode == "f32":
        H.assert_close(gf, gf_ref, RTOL, 1e-7, "feature gradients")
    else:
        H.assert_close(gf.astype(np.float32), gf_ref.astype(np.float32), 2e-3, 1e-7, "feature gradients (fp16)")
    H.assert_close(go, go_ref, RTOL, 2e-7, "opacity gradients")


@pytest.mark.parametrize("tile", [8, 16])
def test_inference_raw37_and_preextracted(gpu, oracle, tile):
    n = 50000
    hv = synthetic.rotated_camera(199, 140, 180.0, 2.5, yaw=-0.4, pitch=0.2)
    pos = synthetic.cube_points(n, 1.5, 41)
    rng = np.random.default_rng(42)
    raw = np.concatenate([rng.normal(-1.0, 1.0, (n, 1)), synthetic.sh_features(n, 43).astype(np.float64)], axis=1)
    raw = raw.astype(np.float16)
    run = H.RasterRun(hv, pos, raw, None, tile, 4, _lib.FEAT_RAW37_F16, inference=True).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_RAW37_F16, inference=True)
    ref = oracle.raster_forward(cfg, pos, raw, None, hv.w2c, hv.position, debug=True)
    dbg = run.debug()
    check_structure(dbg, ref)
    vis = ref["n_touched"] > 0
    H.assert_close(dbg["opacity"][vis], ref["opacity"][vis], RTOL, 1e-6, "activated opacity")
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], 2e-4, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], 2e-4, 1e-6, "alpha")
    H.assert_close(out["depth_image"], ref["depth_image"], 2e-4, 1e-5, "depth image")

    feats = synthetic.sh_features(n, 44)
    _, opac = synthetic.point_attributes(n, 4, "normal", 45)
    run = H.RasterRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_SH36_F16, inference=True).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_SH36_F16, inference=True)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, hv.position)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["depth_image"], ref["depth_image"], RTOL, 1e-5, "depth image")


def test_inference_direct_f16_16_channels(gpu, oracle):
    n = 80000
    hv, pos, feats, opac = scene(n, 16, seed=51, dtype=np.float16)
    run = H.RasterRun(hv, pos, feats, opac, 16, 16, _lib.FEAT_DIRECT_F16, inference=True).forward()
    cfg = oracle_cfg(oracle, hv, n, 16, 16, oracle.FEAT_DIRECT_F16, inference=True)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    check_structure(run.debug(), ref)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["depth_image"], ref["depth_image"], RTOL, 1e-5, "depth image")


@pytest.mark.parametrize("tile", [8, 16])
def test_edge_cases(gpu, oracle, tile):
    hv = synthetic.camera_on_z(64, 48, 50.0, 2.0)

    def compare(pos, what):
        pos = np.asarray(pos, np.float32).reshape(-1, 3)
        n = len(pos)
        feats, opac = synthetic.point_attributes(max(n, 1), 4, "uniform", 3)
        feats, opac = feats[:n], opac[:n]
        run = H.RasterRun(hv, pos, feats if n else np.zeros((0, 4), np.float32), opac if n else np.zeros(0, np.float32),
                          tile, 4, _lib.FEAT_DIRECT_F32).forward()
        ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_DIRECT_F32), pos, feats, opac,
                                    hv.w2c, debug=True)
        if n:
            check_structure(run.debug(), ref)
        out = run.outputs()
        H.assert_close(out["image"], ref["image"], RTOL, 1e-6, what + ": image")
        H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, what + ": alpha")
        if n:
            H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, what + ": weights")
        return ref

    ref = compare(np.zeros((0, 3)), "empty")
    assert (ref["image"] == 0).all()
    ref = compare([[0, 0, -5.0], [0, 0, 200.0], [50.0, 0, 0]], "all culled")
    assert ref["n_visible"] == 0
    compare([[0.0, 0.0, 0.0]], "single point")
    # a plane of points at one depth: every depth key ties, order must fall back to the point id
    g = np.stack(np.meshgrid(np.linspace(-1.2, 1.2, 90), np.linspace(-0.9, 0.9, 70)), -1).reshape(-1, 2)
    plane = np.concatenate([g, np.zeros((len(g), 1))], axis=1)
    ref = compare(np.concatenate([plane, plane[::-1]]), "coplanar points")
    assert ref["n_visible"] > 5000
    # points that project exactly onto pixel centres, pixel corners and tile edges
    px = np.array([0.5, 1.0, 7.5, 8.0, 8.5, 15.5, 16.0, 16.5, 31.5, 32.0, 63.5, 64.0, -0.4, -0.5, 64.4, 64.5])
    xs, ys = np.meshgrid(px, px[:12] * 0.75)
    z = 0.0
    depth = 2.0
    wx = (xs.ravel() - 32.0) / 50.0 * depth
    wy = (ys.ravel() - 24.0) / 50.0 * depth
    compare(np.stack([wx, wy, np.full_like(wx, z)], 1), "pixel / tile boundaries")


@pytest.mark.parametrize("seed,n,width,height,tile,channels", [(70001, 20000, 233, 151, 8, 8), (70002, 2000, 37, 211, 16, 4),
                                                              (70003, 50, 15, 19, 16, 8)])
def test_non_finite_and_extreme_positions(gpu, oracle, seed, n, width, height, tile, channels):
    # NaN, infinite, huge and denormal coordinates, depths on and next to zero and the clipping planes: such points are
    # culled or drawn exactly as the oracle does it (the comparisons of kernels.cu:52-60 with NaN false), nothing
    # overflows a conversion to an integer, and the gradients of the points that are drawn are unaffected
    hv = synthetic.camera_on_z(width, height, 120.0, 2.2)
    pos = H.extreme_positions(hv, n, seed)
    feats, opac = synthetic.point_attributes(n, channels, "normal", seed + 1)
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    check_structure(run.debug(), ref)
    assert 0 < ref["n_visible"] < n
    out = run.outputs()
    assert np.isfinite(out["image"]).all()
    H.assert_close(out["image"], ref["image"], RTOL, 2e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    rng = np.random.default_rng(seed)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
    assert np.isfinite(gf).all() and np.isfinite(go).all()
    H.assert_close(gf, gf_ref, RTOL, 2e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, 2e-6, "opacity gradients")


@pytest.mark.parametrize("tile", [8, 16])
@pytest.mark.parametrize("levels", [40000, 2500, 400, 30], ids=lambda v: f"{v}depths")
def test_runs_of_equal_depth_keys(gpu, oracle, tile, levels):
    # Depths from a set of `levels` values: in a tile of some thousand instances that gives hardly any ties, many runs
    # of two or three equal keys, runs around the length up to which the tile sort puts ties right in place (16), or
    # runs of hundreds (sorted again over the point indices). The instance order inside a run is by point index.
    n, channels = 60000, 4
    hv = synthetic.camera_on_z(64, 48, 50.0, 3.0)
    rng = np.random.default_rng(levels)
    depth = 3.0 + rng.integers(0, levels, n) / levels          # camera space, 3 .. 4
    u, v = rng.uniform(0, 64, n), rng.uniform(0, 48, n)
    pos = np.stack([(u - 32.0) / 50.0 * depth, (v - 24.0) / 50.0 * depth, depth - 3.0], 1).astype(np.float32)
    feats, opac = synthetic.point_attributes(n, channels, "uniform", 5)
    opac *= 0.01
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
    ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32), pos, feats, opac,
                                hv.w2c, debug=True)
    dbg = run.debug()
    check_structure(dbg, ref)
    keys, ranges = dbg["instance_depth_keys"], dbg["tile_ranges"].astype(np.int64)
    same = keys[1:] == keys[:-1]
    same[ranges[1:, 0][ranges[1:, 0] < len(keys)] - 1] = False     # a run ends with its tile
    if levels == 40000:
        assert 0 < same.mean() < 0.2
    elif levels == 30:
        assert same.mean() > 0.9
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")


def test_too_many_tiles_is_rejected(gpu):
    # 65,536 tiles are the reference's limit (16-bit tile key, kernels.cu:204,214); one more is refused
    hv = synthetic.camera_on_z(8 * 257, 8 * 256, 500.0, 3.0)
    with pytest.raises(_lib.BackendError, match="16-bit tile key"):
        H.RasterRun(hv, np.zeros((4, 3), np.float32), np.zeros((4, 4), np.float32), np.ones(4, np.float32), 8, 4,
                    _lib.FEAT_DIRECT_F32)
    hv = synthetic.camera_on_z(8 * 256, 8 * 256, 500.0, 3.0)   # exactly 65,536
    run = H.RasterRun(hv, np.zeros((4, 3), np.float32), np.zeros((4, 4), np.float32), np.ones(4, np.float32), 8, 4,
                      _lib.FEAT_DIRECT_F32)
    assert run.layout.n_tiles == 65536


@pytest.mark.parametrize("width,height,focal", [(1920, 1080, 1500.0), (2473, 1643, 2000.0)],
                         ids=["1920x1080", "2473x1643"])
def test_reference_tile_size_on_large_images(gpu, oracle, width, height, focal):
    # the reference's 8x8 tiles on images of more than 16,384 tiles (32,400 and 63,860): per-tile counters as 16-bit
    # halves in LDS; structure bit-exact, images and gradients to tolerance
    n, channels = 300000, 4
    hv = synthetic.camera_on_z(width, height, focal, 2.6)
    pos = synthetic.cube_points(n, 2.4, 71)
    feats, opac = synthetic.point_attributes(n, channels, "normal", 72)
    run = H.RasterRun(hv, pos, feats, opac, 8, channels, _lib.FEAT_DIRECT_F32).forward()
    assert run.layout.n_tiles > 16384
    cfg = oracle_cfg(oracle, hv, n, 8, channels, oracle.FEAT_DIRECT_F32)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    dbg = run.debug()
    assert dbg["n_visible"] > 0.5 * n
    check_structure(dbg, ref)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    rng = np.random.default_rng(73)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
    H.assert_close(gf, gf_ref, RTOL, 1e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, 2e-7, "opacity gradients")


def test_instances_beyond_the_capacity_are_reported_and_nothing_is_drawn(gpu, oracle):
    # every point on a tile corner: four instances per point, more than a capacity of 2 N holds
    n, tile = 5000, 16
    hv = synthetic.camera_on_z(320, 240, 300.0, 3.0)
    c = hv.camera
    rng = np.random.default_rng(5)
    z = rng.uniform(0.5, 2.0, n).astype(np.float32)
    gx, gy = rng.integers(1, 320 // tile, n), rng.integers(1, 240 // tile, n)
    wx = ((gx * tile - c.center_x) / c.focal_x * (z + 3.0)).astype(np.float32)
    wy = ((gy * tile - c.center_y) / c.focal_y * (z + 3.0)).astype(np.float32)
    pos = np.stack([wx, wy, z], 1)
    feats, opac = synthetic.point_attributes(n, 4, "normal", 6)
    cfg = oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_DIRECT_F32)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    assert ref["n_instances"] > 3 * n
    small = H.RasterRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_DIRECT_F32, max_instances=2 * n).forward()
    assert small.layout.max_instances == 2 * n
    with pytest.raises(_lib.BackendError, match="do not fit max_instances"):
        small.counters()
    out = small.outputs()
    assert (out["image"] == 0).all() and (out["alpha"] == 0).all() and (out["blending_weights"] == 0).all()
    gf, go = small.backward(np.ones_like(ref["image"]), np.ones_like(ref["alpha"]))
    assert (gf == 0).all() and (go == 0).all()
    # the same workspace size is enough for a call that fits, and a capacity of 4 N always is
    run = H.RasterRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_DIRECT_F32).forward()
    check_structure(run.debug(), ref)
    H.assert_close(run.outputs()["image"], ref["image"], RTOL, 1e-5, "image")


def test_operator_layer_grows_the_workspace_when_the_default_capacity_is_exceeded(gpu, oracle, monkeypatch):
    from inpc_amd import rasterization, rasterize_points

    n, tile = 5000, 16
    hv = synthetic.camera_on_z(320, 240, 300.0, 3.0)
    c = hv.camera
    rng = np.random.default_rng(8)
    z = rng.uniform(0.5, 2.0, n).astype(np.float32)
    gx, gy = rng.integers(1, 320 // tile, n), rng.integers(1, 240 // tile, n)
    pos = np.stack([((gx * tile - c.center_x) / c.focal_x * (z + 3.0)).astype(np.float32),
                    ((gy * tile - c.center_y) / c.focal_y * (z + 3.0)).astype(np.float32), z], 1)
    feats, opac = synthetic.point_attributes(n, 4, "normal", 9)
    monkeypatch.setattr(rasterization, "_ALWAYS_FITS_POINTS", 0)   # take the library's default capacity
    image, alpha, weights = rasterize_points(hv.to_view(gpu), H.dev(pos), H.dev(feats), H.dev(opac), tile=tile)
    ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, tile, 4, oracle.FEAT_DIRECT_F32), pos, feats, opac, hv.w2c)
    H.assert_close(image.cpu().numpy(), ref["image"], RTOL, 1e-5, "image")
    H.assert_close(weights.cpu().numpy(), ref["blending_weights"], RTOL, 1e-7, "blending weights")


def test_autograd_api_sh_and_direct(gpu, oracle):
    from inpc_amd import INPCRasterizer, rasterize_points

    n = 30000
    hv = synthetic.camera_on_z(160, 120, 140.0, 2.5)
    view = hv.to_view(gpu)
    pos = synthetic.cube_points(n, 1.5, 61)
    feats = synthetic.sh_features(n, 62)
    _, opac = synthetic.point_attributes(n, 4, "normal", 63)
    positions = H.dev(pos)
    features = H.dev(feats).requires_grad_(True)
    opacities = H.dev(opac.reshape(-1, 1)).requires_grad_(True)
    rasterizer = INPCRasterizer()
    image, alpha, weights = rasterizer(view, 0, positions, features, opacities)
    assert image.shape == (4, 120, 160) and alpha.shape == (1, 120, 160) and weights.shape == (n,)
    assert not weights.requires_grad
    cfg = oracle_cfg(oracle, hv, n, 8, 4, oracle.FEAT_SH36_F16)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, hv.position)
    H.assert_close(image.detach().cpu().numpy(), ref["image"], RTOL, 1e-5, "image")
    # only the image is used: grad_alpha arrives as None and must be treated as zero
    gi = torch.randn_like(image) * 1e-2
    (image * gi).sum().backward()
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi.cpu().numpy(), np.zeros_like(ref["alpha"]),
                                               image.detach().cpu().numpy(), alpha.detach().cpu().numpy(), pos, feats,
                                               opac, hv.w2c, hv.position)
    assert features.grad.shape == (n, 36) and features.grad.dtype == torch.float16
    assert opacities.grad.shape == (n, 1)
    H.assert_close(features.grad.float().cpu().numpy(), gf_ref.astype(np.float32), 2e-3, 1e-7, "SH gradients")
    H.assert_close(opacities.grad.cpu().numpy().reshape(-1), go_ref, RTOL, 1e-7, "opacity gradients")

    # render / render_preextracted return (image, depth, alpha)
    img2, depth2, alpha2 = rasterizer.render_preextracted(view, 0, positions, features.detach(), opacities.detach())
    H.assert_close(img2.cpu().numpy(), ref["image"], RTOL, 1e-5, "preextracted image")
    assert depth2.shape == (1, 120, 160)

    f8, o8 = synthetic.point_attributes(n, 8, "normal", 64)
    f8d = H.dev(f8).requires_grad_(True)
    o8d = H.dev(o8).requires_grad_(True)
    image8, alpha8, w8 = rasterize_points(view, positions, f8d, o8d, tile=16)
    (image8.sum() + alpha8.sum()).backward()
    cfg8 = oracle_cfg(oracle, hv, n, 16, 8, oracle.FEAT_DIRECT_F32)
    ref8 = oracle.raster_forward(cfg8, pos, f8, o8, hv.w2c)
    ones_i, ones_a = np.ones_like(ref8["image"]), np.ones_like(ref8["alpha"])
    gf8, go8, _ = oracle.raster_backward(cfg8, ones_i, ones_a, image8.detach().cpu().numpy(),
                                         alpha8.detach().cpu().numpy(), pos, f8, o8, hv.w2c)
    H.assert_close(f8d.grad.cpu().numpy(), gf8, RTOL, 1e-6, "direct feature gradients")
    H.assert_close(o8d.grad.cpu().numpy(), go8, RTOL, 1e-5, "direct opacity gradients")


@pytest.mark.parametrize("tile", [8, 16])
def test_backward_twice_after_one_forward(gpu, oracle, tile):
    # The gradient rows of points that straddle tiles carry flags from one backward call to the next: a second
    # call with gradients that vanish on half of the image (so that fewer rows are written) must not see the
    # first call's rows. Dense and opaque, so that tiles also end early.
    n, channels = 120000, 8
    hv = synthetic.camera_on_z(131, 93, 120.0, 2.4)
    pos = synthetic.cube_points(n, 1.3, 41)
    feats, _ = synthetic.point_attributes(n, channels, "normal", 42)
    opac = np.random.default_rng(43).uniform(0.05, 0.9, n).astype(np.float32)
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32)
    out = run.outputs()
    rng = np.random.default_rng(44)
    for half in (False, True):
        gi = rng.normal(0, 1e-2, out["image"].shape).astype(np.float32)
        ga = rng.normal(0, 1e-2, out["alpha"].shape).astype(np.float32)
        if half:
            gi[:, :, : gi.shape[2] // 2] = 0.0
            ga[:, :, : ga.shape[2] // 2] = 0.0
        gf, go = run.backward(gi, ga)
        gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
        H.assert_close(gf, gf_ref, RTOL, 1e-7, f"feature gradients (half={half})")
        H.assert_close(go, go_ref, RTOL, 2e-7, f"opacity gradients (half={half})")


RANDOM_CASES = [
    # seed, n, width, height, focal, tile, channels, opacity range, cluster share
    (101, 9000, 37, 29, 40.0, 8, 4, (0.0, 1.0), 0.0),
    (102, 30000, 130, 71, 110.0, 16, 8, (0.0, 0.2), 0.3),
    (103, 20000, 65, 65, 70.0, 16, 4, (0.9, 1.0), 0.5),
    (104, 25000, 129, 33, 95.0, 8, 8, (0.3, 0.7), 0.8),
    (105, 12000, 16, 16, 30.0, 16, 16, (0.0, 0.6), 0.2),
    (106, 40000, 200, 120, 150.0, 8, 16, (0.01, 0.05), 0.6),
]


@pytest.mark.parametrize("case", RANDOM_CASES, ids=[f"seed{c[0]}" for c in RANDOM_CASES])
def test_random_scenes_forward_backward(gpu, oracle, case):
    # Odd image sizes, clusters of hundreds of points on single pixels (long per-pixel lists across several batches,
    # early termination), opacities at exactly 0 and 1, points on tile borders: forward and backward against the oracle.
    seed, n, width, height, focal, tile, channels, (lo, hi), cluster = case
    rng = np.random.default_rng(seed)
    hv = synthetic.camera_on_z(width, height, focal, 2.4)
    pos = synthetic.cube_points(n, 1.4, seed)
    n_cluster = int(n * cluster)
    if n_cluster:
        spots = rng.uniform(-0.5, 0.5, (7, 3)).astype(np.float32)
        pos[:n_cluster] = spots[rng.integers(0, 7, n_cluster)] + rng.normal(0, 2e-3, (n_cluster, 3)).astype(np.float32)
    feats, _ = synthetic.point_attributes(n, channels, "normal", seed + 1)
    opac = rng.uniform(lo, hi, n).astype(np.float32)
    opac[::97] = 0.0
    if hi >= 1.0:
        opac[5::89] = 1.0
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    check_structure(run.debug(), ref)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 2e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
    H.assert_close(gf, gf_ref, RTOL, 2e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, 2e-6, "opacity gradients")


@pytest.mark.real_gpu
def test_forward_backward_replays_from_a_graph(gpu, oracle):
    # The library enqueues kernels only (no allocation, no memset nodes, no host read-back in forward / backward),
    # so a caller may capture a step into a graph. Replays with new inputs written in place must give what eager
    # calls give; the replays are interleaved with eager work and synchronisations.
    n, channels, tile = 30000, 8, 16
    hv, pos, feats, opac = scene(n, channels, seed=77)
    run = H.RasterRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32)
    lib = _lib.lib()
    gf = torch.empty((n, channels), dtype=torch.float32, device=gpu)
    go = torch.empty((n,), dtype=torch.float32, device=gpu)
    Hh, Ww = hv.camera.height, hv.camera.width
    gi = torch.zeros((channels, Hh, Ww), dtype=torch.float32, device=gpu)
    ga = torch.zeros((1, Hh, Ww), dtype=torch.float32, device=gpu)

    def step():
        s = _lib.current_stream()
        _lib.check(lib.inpc_raster_forward(
            C.byref(run.cfg), _lib.ptr(run.positions), _lib.ptr(run.features), _lib.ptr(run.opacities), _lib.ptr(run.w2c),
            _lib.ptr(run.cam_position), _lib.ptr(run.image), _lib.ptr(run.alpha), _lib.ptr(run.bw), None,
            _lib.ptr(run.ws), run.layout.total_bytes, s), "forward")
        _lib.check(lib.inpc_raster_backward(
            C.byref(run.cfg), _lib.ptr(gi), _lib.ptr(ga), _lib.ptr(run.image), _lib.ptr(run.alpha), _lib.ptr(run.positions),
            _lib.ptr(run.cam_position), _lib.ptr(gf), _lib.ptr(go), None, _lib.ptr(run.ws), run.layout.total_bytes, s),
            "backward")

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        step()   # warm-up outside the capture (function attributes, occupancy queries)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    rng = np.random.default_rng(78)
    cfg = oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32)
    for replay in range(3):
        new_pos = synthetic.cube_points(n, 1.6, 200 + replay)
        new_feats, new_opac = synthetic.point_attributes(n, channels, "normal", 300 + replay, np.float32)
        new_gi = rng.normal(0, 1e-2, (channels, Hh, Ww)).astype(np.float32)
        new_ga = rng.normal(0, 1e-2, (1, Hh, Ww)).astype(np.float32)
        run.positions.copy_(H.dev(new_pos))
        run.features.copy_(H.dev(new_feats))
        run.opacities.copy_(H.dev(new_opac))
        gi.copy_(H.dev(new_gi))
        ga.copy_(H.dev(new_ga))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = oracle.raster_forward(cfg, new_pos, new_feats, new_opac, hv.w2c)
        out = run.outputs()
        H.assert_close(out["image"], ref["image"], RTOL, 1e-5, f"image, replay {replay}")
        H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, f"blending weights, replay {replay}")
        gf_ref, go_ref, _ = oracle.raster_backward(cfg, new_gi, new_ga, out["image"], out["alpha"], new_pos, new_feats,
                                                   new_opac, hv.w2c)
        H.assert_close(gf.cpu().numpy(), gf_ref, RTOL, 1e-7, f"feature gradients, replay {replay}")
        H.assert_close(go.cpu().numpy(), go_ref, RTOL, 2e-7, f"opacity gradients, replay {replay}")
