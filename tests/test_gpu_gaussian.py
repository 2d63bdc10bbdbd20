"""GPU parity of the rasterizer's Gaussian footprint against the CPU oracle, through the C ABI.

Bit-exact: tile bounds, screen coordinates, conics, depth order, instance order, tile ranges, and (because the
footprint's exponential is one fixed sequence of fp32 operations on both sides) image, alpha and depth image.
Within 1e-4 relative: blending weights and gradients, which both sides sum in an order of their own. The opacity
gradient contains the difference between the running and the final pixel value, which cancels towards the end of a
pixel's list; the kernel carries that difference as one scalar, the oracle per channel as the reference writes it,
so small elements differ by more than 1e-4 of themselves: the comparison has an absolute floor of 2e-6 (`grad_atol`).
"""
import numpy as np
import pytest
import torch

from inpc_amd import _lib, synthetic
from tests import helpers as H
from tests.test_oracle_gaussian import gcfg_of, near_camera_points

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def grad_atol(ref):
    """Absolute floor of a gradient comparison: 2e-7 for feature gradients, 2e-6 for opacity gradients (the same
    floors as for the bilinear footprint)."""
    return 2e-7 if np.asarray(ref).ndim == 2 else 2e-6


def oracle_run(O, hv, pos, feats, opac, tile, channels, mode=None, inference=False, scales=None, sigma_world=0.0,
               sigma_cutoff=3.0, cam_position=None):
    n = len(pos)
    g = gcfg_of(O, hv, n, tile, channels, mode, inference, sigma_world, sigma_cutoff)
    count = O.gaussian_instance_count(g, pos, hv.w2c, scales)
    ref = O.raster_forward(g.base, pos, feats, opac, hv.w2c, cam_position, debug=True, gaussian=g, scales=scales,
                           n_instances_hint=count)
    return g, ref


def check_structure(dbg, ref):
    assert dbg["n_visible"] == ref["n_visible"]
    assert dbg["n_instances"] == ref["n_instances"]
    np.testing.assert_array_equal(dbg["n_touched"], ref["n_touched"])
    np.testing.assert_array_equal(dbg["bounds"], ref["bounds"])
    for name in ("screen_xy", "conic", "depth"):
        np.testing.assert_array_equal(dbg[name].view(np.uint32), ref[name].view(np.uint32), err_msg=name)
    np.testing.assert_array_equal(dbg["depth_keys"], ref["depth_keys"])
    np.testing.assert_array_equal(dbg["depth_order"], ref["depth_order"])
    np.testing.assert_array_equal(dbg["instance_keys"], ref["instance_keys"])
    np.testing.assert_array_equal(dbg["instance_points"], ref["instance_points"])
    np.testing.assert_array_equal(dbg["tile_ranges"], ref["tile_ranges"])


def scene(n, channels, seed, width=251, height=163, focal=230.0, near=400):
    hv = synthetic.rotated_camera(width, height, focal, 2.4, 0.2, -0.1)
    pos = synthetic.cube_points(n, 1.6, seed)
    if near:
        pos[:near] = near_camera_points(hv, near, seed + 7)   # footprints of many tiles
    feats, opac = synthetic.point_attributes(n, channels, "normal", seed + 1)
    return hv, pos, feats, opac


@pytest.mark.parametrize("tile", [8, 16])
@pytest.mark.parametrize("channels", [4, 8, 16])
def test_forward_direct_f32(gpu, oracle, tile, channels):
    n = 40000
    hv, pos, feats, opac = scene(n, channels, seed=tile + channels)
    run = H.GaussianRun(hv, pos, feats, opac, tile, channels).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels)
    assert ref["n_touched"].max() > 16
    dbg = run.debug()
    check_structure(dbg, ref)
    np.testing.assert_array_equal(dbg["features_view"], ref["features_view"])
    out = run.outputs()
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")


@pytest.mark.parametrize("tile", [8, 16])
def test_forward_backward_dense_opaque_scene(gpu, oracle, tile):
    # many nearly opaque points per pixel: early termination, tiles of many batches
    n = 120000
    hv = synthetic.camera_on_z(97, 61, 90.0, 2.4)
    pos = synthetic.cube_points(n, 1.2, 5)
    feats, _ = synthetic.point_attributes(n, 8, "uniform", 6)
    opac = np.random.default_rng(7).uniform(0.3, 0.999, n).astype(np.float32)
    run = H.GaussianRun(hv, pos, feats, opac, tile, 8).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, 8)
    check_structure(run.debug(), ref)
    out = run.outputs()
    assert (ref["alpha"] == 1.0).mean() > 0.3
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    rng = np.random.default_rng(8)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                               gaussian=g)
    H.assert_close(gf, gf_ref, RTOL, 1e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, grad_atol(go_ref), "opacity gradients")


@pytest.mark.real_gpu
def test_forward_backward_replay_from_a_graph_with_new_inputs(gpu, oracle):
    # A captured step keeps its kernel arguments, so whatever tells this pass's gradient rows from an earlier
    # pass's has to change on the device. The scene saturates (tiles end early and leave rows unwritten) and has
    # points over several tiles; every replay gets new points in place and is checked against the oracle.
    import ctypes as C
    n, tile, channels = 90000, 8, 8
    hv = synthetic.camera_on_z(97, 61, 90.0, 2.4)
    rng = np.random.default_rng(41)

    def inputs(seed):
        pos = synthetic.cube_points(n, 1.2, seed)
        feats, _ = synthetic.point_attributes(n, channels, "uniform", seed + 1)
        opac = np.random.default_rng(seed + 2).uniform(0.3, 0.999, n).astype(np.float32)
        return pos, feats, opac

    pos, feats, opac = inputs(500)
    run = H.GaussianRun(hv, pos, feats, opac, tile, channels)
    lib = _lib.lib()
    Hh, Ww = hv.camera.height, hv.camera.width
    gf = torch.empty((n, channels), dtype=torch.float32, device=gpu)
    go = torch.empty((n,), dtype=torch.float32, device=gpu)
    gi = torch.zeros((channels, Hh, Ww), dtype=torch.float32, device=gpu)
    ga = torch.zeros((1, Hh, Ww), dtype=torch.float32, device=gpu)

    def step():
        s = _lib.current_stream()
        _lib.check(lib.inpc_gaussian_forward(
            C.byref(run.cfg), _lib.ptr(run.positions), _lib.ptr(run.features), _lib.ptr(run.opacities), None,
            _lib.ptr(run.w2c), _lib.ptr(run.cam_position), _lib.ptr(run.image), _lib.ptr(run.alpha), _lib.ptr(run.bw),
            None, _lib.ptr(run.ws), run.layout.total_bytes, s), "forward")
        _lib.check(lib.inpc_gaussian_backward(
            C.byref(run.cfg), _lib.ptr(gi), _lib.ptr(ga), _lib.ptr(run.image), _lib.ptr(run.alpha),
            _lib.ptr(run.positions), _lib.ptr(run.cam_position), _lib.ptr(gf), _lib.ptr(go), None, _lib.ptr(run.ws),
            run.layout.total_bytes, s), "backward")

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        step()   # warm-up outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    for replay in range(3):
        pos, feats, opac = inputs(510 + 10 * replay)
        new_gi = rng.normal(0, 1e-2, (channels, Hh, Ww)).astype(np.float32)
        new_ga = rng.normal(0, 1e-2, (1, Hh, Ww)).astype(np.float32)
        run.positions.copy_(H.dev(pos))
        run.features.copy_(H.dev(feats))
        run.opacities.copy_(H.dev(opac))
        gi.copy_(H.dev(new_gi))
        ga.copy_(H.dev(new_ga))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels)
        assert (ref["alpha"] == 1.0).mean() > 0.3 and (ref["n_touched"] > 1).mean() > 0.2
        out = run.outputs()
        np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
        np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
        gf_ref, go_ref, _ = oracle.raster_backward(g.base, new_gi, new_ga, ref["image"], ref["alpha"], pos, feats,
                                                   opac, hv.w2c, gaussian=g)
        H.assert_close(gf.cpu().numpy(), gf_ref, RTOL, grad_atol(gf_ref), f"feature gradients, replay {replay}")
        H.assert_close(go.cpu().numpy(), go_ref, RTOL, grad_atol(go_ref), f"opacity gradients, replay {replay}")


@pytest.mark.parametrize("tile", [8, 16])
def test_forward_sh36_and_backward(gpu, oracle, tile):
    n = 30000
    hv = synthetic.rotated_camera(233, 171, 210.0, 2.6, yaw=0.5, pitch=-0.3)
    pos = synthetic.cube_points(n, 1.5, 11)
    pos[:300] = near_camera_points(hv, 300, 3)
    feats = synthetic.sh_features(n, 12)
    _, opac = synthetic.point_attributes(n, 4, "normal", 13)
    run = H.GaussianRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_SH36_F16).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, 4, oracle.FEAT_SH36_F16, cam_position=hv.position)
    dbg = run.debug()
    check_structure(dbg, ref)
    vis = ref["n_touched"] > 0
    H.assert_close(dbg["features_view"][vis], ref["features_view"][vis], RTOL, 1e-5, "SH view features")
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    rng = np.random.default_rng(14)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    image_gpu, alpha_gpu = out["image"], out["alpha"]
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, image_gpu, alpha_gpu, pos, feats, opac, hv.w2c,
                                               hv.position, gaussian=g)
    assert (gf[~vis] == 0).all() and (go[~vis] == 0).all()
    H.assert_close(gf.astype(np.float32), gf_ref.astype(np.float32), 2e-3, 1e-7, "SH gradients")
    H.assert_close(go, go_ref, RTOL, grad_atol(go_ref), "opacity gradients")


@pytest.mark.parametrize("mode", ["f16", "f32"])
def test_backward_direct(gpu, oracle, mode):
    n, tile, channels = 50000, 16, 4
    hv, pos, feats, opac = scene(n, channels, seed=21)
    fmode = _lib.FEAT_DIRECT_F16 if mode == "f16" else _lib.FEAT_DIRECT_F32
    if mode == "f16":
        feats = feats.astype(np.float16)
    run = H.GaussianRun(hv, pos, feats, opac, tile, channels, fmode).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels, fmode)
    check_structure(run.debug(), ref)
    out = run.outputs()
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    rng = np.random.default_rng(22)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                               gaussian=g)
    if mode == "f16":
        H.assert_close(gf.astype(np.float32), gf_ref.astype(np.float32), 2e-3, 1e-7, "feature gradients")
    else:
        H.assert_close(gf, gf_ref, RTOL, 1e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, grad_atol(go_ref), "opacity gradients")


@pytest.mark.parametrize("seed,n,width,height,tile", [(71001, 20000, 233, 151, 8), (71002, 2000, 37, 211, 16)])
def test_non_finite_and_extreme_positions(gpu, oracle, seed, n, width, height, tile):
    # as for the bilinear footprint: NaN, infinite, huge and denormal coordinates, depths on and next to zero and the
    # clipping planes (a depth next to zero makes a footprint of the whole image: kernels.cu:62-70 clamps the bounds)
    channels = 4
    hv = synthetic.camera_on_z(width, height, 120.0, 2.2)
    pos = H.extreme_positions(hv, n, seed)
    feats, opac = synthetic.point_attributes(n, channels, "normal", seed + 1)
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels)
    run = H.GaussianRun(hv, pos, feats, opac, tile, channels, _lib.FEAT_DIRECT_F32,
                        max_instances=max(int(ref["n_instances"]) + 1024, 4 * n)).forward()
    check_structure(run.debug(), ref)
    assert 0 < ref["n_visible"] < n
    out = run.outputs()
    assert np.isfinite(out["image"]).all()
    H.assert_close(out["image"], ref["image"], RTOL, 2e-5, "image")
    rng = np.random.default_rng(seed)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _, audit = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                                      gaussian=g, audit=True)
    assert np.isfinite(gf).all() and np.isfinite(go).all()
    H.assert_gradient_close(gf, audit, "view", "feature gradients")
    H.assert_gradient_close(go, audit, "opacity", "opacity gradients")


@pytest.mark.parametrize("with_scales", [False, True])
@pytest.mark.parametrize("tile", [8, 16])
def test_inference_preextracted(gpu, oracle, tile, with_scales):
    n = 30000
    hv, pos, _, opac = scene(n, 4, seed=31, near=0)
    feats = synthetic.sh_features(n, 32)
    scales = (np.random.default_rng(5).random(n) * 0.01).astype(np.float32) if with_scales else None
    kw = dict(inference=True, scales=scales, sigma_world=0.006, sigma_cutoff=2.5)
    run = H.GaussianRun(hv, pos, feats, opac, tile, 4, _lib.FEAT_SH36_F16, **kw).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, 4, oracle.FEAT_SH36_F16, cam_position=hv.position, **kw)
    check_structure(run.debug(), ref)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["depth_image"], ref["depth_image"], RTOL, 1e-6, "depth image")


def test_inference_raw37(gpu, oracle):
    n, tile = 20000, 8
    hv, pos, _, _ = scene(n, 4, seed=41, near=0)
    rng = np.random.default_rng(42)
    raw = np.concatenate([rng.normal(-1.0, 1.0, (n, 1)), synthetic.sh_features(n, 43).astype(np.float64)], axis=1)
    raw = raw.astype(np.float16)
    kw = dict(inference=True, sigma_world=0.004, sigma_cutoff=3.0)
    run = H.GaussianRun(hv, pos, raw, None, tile, 4, _lib.FEAT_RAW37_F16, **kw).forward()
    g, ref = oracle_run(oracle, hv, pos, raw, None, tile, 4, oracle.FEAT_RAW37_F16, cam_position=hv.position, **kw)
    dbg = run.debug()
    np.testing.assert_array_equal(dbg["instance_points"], ref["instance_points"])
    vis = ref["n_touched"] > 0
    H.assert_close(dbg["opacity"][vis], ref["opacity"][vis], RTOL, 1e-7, "activated opacity")
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], 2e-4, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], 2e-4, 1e-6, "alpha")
    H.assert_close(out["depth_image"], ref["depth_image"], 2e-4, 1e-5, "depth image")


def test_edge_cases(gpu, oracle):
    hv = synthetic.camera_on_z(64, 48, 60.0, 2.0)
    # no points at all: background images
    run = H.GaussianRun(hv, np.zeros((0, 3), np.float32), np.zeros((0, 4), np.float32), np.zeros(0, np.float32)).forward()
    out = run.outputs()
    assert (out["image"] == 0).all() and (out["alpha"] == 0).all()
    # every point behind the camera
    n = 1000
    pos = synthetic.cube_points(n, 1.0, 1)
    pos[:, 2] -= 10.0
    feats, opac = synthetic.point_attributes(n, 4, "uniform", 2)
    run = H.GaussianRun(hv, pos, feats, opac).forward()
    _, counters = run.counters()
    assert counters[:2] == [0, 0]
    out = run.outputs()
    assert (out["image"] == 0).all() and (out["alpha"] == 0).all() and (out["blending_weights"] == 0).all()
    gf, go = run.backward(np.ones((4, 48, 64), np.float32), np.ones((1, 48, 64), np.float32))
    assert (gf == 0).all() and (go == 0).all()
    # a single point
    one = np.array([[0.01, -0.02, 0.0]], np.float32)
    run = H.GaussianRun(hv, one, np.ones((1, 4), np.float32), np.array([0.7], np.float32)).forward()
    g, ref = oracle_run(oracle, hv, one, np.ones((1, 4), np.float32), np.array([0.7], np.float32), 8, 4)
    np.testing.assert_array_equal(run.outputs()["image"].view(np.uint32), ref["image"].view(np.uint32))


@pytest.mark.parametrize("width,height,focal", [(1920, 1080, 1500.0), (2473, 1643, 2000.0)],
                         ids=["1920x1080", "2473x1643"])
def test_reference_tile_size_on_large_images(gpu, oracle, width, height, focal):
    # 8x8 tiles on images of more than 16,384 tiles (32,400 and 63,860): the bins are counted and filled in windows
    # of 32,768 tiles by blocks of 1024 threads; footprints that straddle the windows come from the near points
    n, channels = 200000, 4
    hv, pos, feats, opac = scene(n, channels, seed=81, width=width, height=height, focal=focal, near=300)   # the first 300
    run = H.GaussianRun(hv, pos, feats, opac, 8, channels, _lib.FEAT_DIRECT_F32).forward()
    assert run.layout.n_tiles > 16384
    g, ref = oracle_run(oracle, hv, pos, feats, opac, 8, channels)
    dbg = run.debug()
    assert dbg["n_visible"] > 0.5 * n
    check_structure(dbg, ref)
    out = run.outputs()
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    rng = np.random.default_rng(82)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _, audit = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac,
                                                      hv.w2c, gaussian=g, audit=True)
    # The near points cover up to thousands of pixels in dozens of tiles at this focal length: their gradients are sums
    # of that many terms of both signs, some of them orders of magnitude smaller than their terms. One bound for every
    # point: 1e-4 of the sum taken in double precision plus kGradUnits rounding units of the sum of the magnitudes
    # (tests/helpers.py); the oracle's own fp32 sums are held to the same bound.
    H.assert_gradient_close(gf, audit, "view", "feature gradients")
    H.assert_gradient_close(go, audit, "opacity", "opacity gradients")
    H.assert_gradient_close(gf_ref, audit, "view", "the oracle's fp32 feature gradients")
    H.assert_gradient_close(go_ref, audit, "opacity", "the oracle's fp32 opacity gradients")
    # and the points with small footprints also against the fp32 oracle directly
    near = 300
    H.assert_close(gf[near:], gf_ref[near:], RTOL, grad_atol(gf_ref), "feature gradients")
    H.assert_close(go[near:], go_ref[near:], RTOL, grad_atol(go_ref), "opacity gradients")


@pytest.mark.parametrize("tile,channels", [(8, 4), (16, 8), (16, 16)])
def test_gradients_are_the_same_bits_on_every_run(gpu, oracle, tile, channels):
    # Footprints of many pixels and many tiles, added up without float atomics: per instance the pixels' shares in a
    # fixed order (lanes, then waves), per point the instances' rows in row order. Three forward + backward passes,
    # each in a workspace of its own with other stale bytes, must agree bit for bit.
    n = 30000
    hv, pos, feats, opac = scene(n, channels, seed=90 + tile + channels, near=2000)
    rng = np.random.default_rng(91)
    results = []
    for _ in range(3):
        run = H.GaussianRun(hv, pos, feats, opac, tile, channels).forward()
        out = run.outputs()
        if not results:
            gi = rng.normal(0, 1e-2, out["image"].shape).astype(np.float32)
            ga = rng.normal(0, 1e-2, out["alpha"].shape).astype(np.float32)
        gf, go = run.backward(gi, ga)
        results.append((gf.copy(), go.copy()))
    assert np.abs(results[0][0]).max() > 0
    for gf, go in results[1:]:
        np.testing.assert_array_equal(gf.view(np.uint32), results[0][0].view(np.uint32))
        np.testing.assert_array_equal(go.view(np.uint32), results[0][1].view(np.uint32))
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels)
    _, _, _, audit = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                            gaussian=g, audit=True)
    H.assert_gradient_close(results[0][0], audit, "view", "feature gradients")
    H.assert_gradient_close(results[0][1], audit, "opacity", "opacity gradients")


def test_instances_beyond_the_capacity_are_reported(gpu, oracle):
    n = 5000
    hv, pos, feats, opac = scene(n, 4, seed=51, near=500)
    g, ref = oracle_run(oracle, hv, pos, feats, opac, 8, 4)
    need = ref["n_instances"]
    small = H.GaussianRun(hv, pos, feats, opac, 8, 4, max_instances=need - 1).forward()
    rc, counters = small.counters(check=False)
    assert rc == -2 and counters[1] == need and counters[3] == 0      # INPC_E_WORKSPACE, nothing drawn
    out = small.outputs()
    assert (out["image"] == 0).all() and (out["alpha"] == 0).all()
    # the backward pass of a call that drew nothing gives zero gradients
    gf, go = small.backward(np.ones_like(out["image"]), np.ones_like(out["alpha"]))
    assert (gf == 0).all() and (go == 0).all()
    exact = H.GaussianRun(hv, pos, feats, opac, 8, 4, max_instances=need).forward()
    rc, counters = exact.counters()
    assert counters[1] == need and counters[3] == need
    np.testing.assert_array_equal(exact.outputs()["image"].view(np.uint32), ref["image"].view(np.uint32))


def test_python_api(gpu, oracle):
    from inpc_amd import INPCRasterizer, rasterize_points

    n = 20000
    hv = synthetic.rotated_camera(160, 120, 140.0, 2.5, 0.3, 0.1)
    view = hv.to_view(gpu)
    pos = synthetic.cube_points(n, 1.5, 61)
    pos[:200] = near_camera_points(hv, 200, 5)
    feats = synthetic.sh_features(n, 62)
    _, opac = synthetic.point_attributes(n, 4, "normal", 63)
    rasterizer = INPCRasterizer()
    positions = H.dev(pos)
    features = H.dev(feats).requires_grad_(True)
    opacities = H.dev(opac.reshape(-1, 1)).requires_grad_(True)
    image, alpha, weights = rasterizer(view, 1, positions, features, opacities)
    g, ref = oracle_run(oracle, hv, pos, feats, opac, 8, 4, oracle.FEAT_SH36_F16, cam_position=hv.position)
    H.assert_close(image.detach().cpu().numpy(), ref["image"], RTOL, 1e-5, "image")
    H.assert_close(weights.cpu().numpy(), ref["blending_weights"], RTOL, 1e-7, "blending weights")
    (image.sum() + alpha.sum()).backward()
    ones_i, ones_a = np.ones_like(ref["image"]), np.ones_like(ref["alpha"])
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, ones_i, ones_a, image.detach().cpu().numpy(),
                                               alpha.detach().cpu().numpy(), pos, feats, opac, hv.w2c, hv.position,
                                               gaussian=g)
    H.assert_close(features.grad.float().cpu().numpy(), gf_ref.astype(np.float32), 2e-3, 1e-6, "SH gradients")
    H.assert_close(opacities.grad.cpu().numpy().reshape(-1), go_ref, RTOL, grad_atol(go_ref), "opacity gradients")
    # render_preextracted: sigma_world = scale * 0.05 / focal_y (B/torch_bindings/rasterization.py:130-134)
    img2, depth2, alpha2 = rasterizer.render_preextracted(view, 1, positions, features.detach(), opacities.detach(),
                                                          None, 2.0, 2.5)
    g2, ref2 = oracle_run(oracle, hv, pos, feats, opac, 8, 4, oracle.FEAT_SH36_F16, inference=True,
                          sigma_world=float(np.float32(2.0 * 0.05 / hv.camera.focal_y)), sigma_cutoff=2.5,
                          cam_position=hv.position)
    H.assert_close(img2.cpu().numpy(), ref2["image"], RTOL, 1e-5, "preextracted image")
    H.assert_close(depth2.cpu().numpy(), ref2["depth_image"], RTOL, 1e-6, "preextracted depth")
    # a second call with far more instances than the default buffers hold: the wrapper sizes them and goes again
    pos_near = near_camera_points(hv, 10000, 9)
    f8, o8 = synthetic.point_attributes(10000, 8, "normal", 64)
    img8, alpha8, w8 = rasterize_points(view, H.dev(pos_near), H.dev(f8), H.dev(o8), tile=8, mode=1)
    g8, ref8 = oracle_run(oracle, hv, pos_near, f8, o8, 8, 8)
    assert ref8["n_instances"] > 4 * 10000 + 65536
    np.testing.assert_array_equal(img8.cpu().numpy().view(np.uint32), ref8["image"].view(np.uint32))


RANDOM_CASES = [
    # seed, n, width, height, focal, tile, channels, opacity range, cluster share, share of points close to the camera
    (201, 9000, 37, 29, 40.0, 8, 4, (0.0, 1.0), 0.0, 0.0),
    (202, 30000, 130, 71, 110.0, 16, 8, (0.0, 0.2), 0.3, 0.01),
    (203, 20000, 65, 65, 70.0, 16, 4, (0.9, 1.0), 0.5, 0.0),
    (204, 25000, 129, 33, 95.0, 8, 8, (0.3, 0.7), 0.8, 0.02),
    (205, 12000, 16, 16, 30.0, 16, 16, (0.0, 0.6), 0.2, 0.05),
    (206, 40000, 200, 120, 150.0, 8, 16, (0.01, 0.05), 0.6, 0.0),
]


@pytest.mark.parametrize("case", RANDOM_CASES, ids=[f"seed{c[0]}" for c in RANDOM_CASES])
def test_random_scenes_forward_backward(gpu, oracle, case):
    # Odd image sizes, clusters of hundreds of points on single pixels (long per-pixel lists over several batches,
    # early termination), opacities at exactly 0 and 1, footprints with and without slots side by side.
    seed, n, width, height, focal, tile, channels, (lo, hi), cluster, near = case
    rng = np.random.default_rng(seed)
    hv = synthetic.camera_on_z(width, height, focal, 2.4)
    pos = synthetic.cube_points(n, 1.4, seed)
    n_cluster = int(n * cluster)
    if n_cluster:
        spots = rng.uniform(-0.5, 0.5, (7, 3)).astype(np.float32)
        pos[:n_cluster] = spots[rng.integers(0, 7, n_cluster)] + rng.normal(0, 2e-3, (n_cluster, 3)).astype(np.float32)
    n_near = int(n * near)
    if n_near:
        pos[n - n_near:] = near_camera_points(hv, n_near, seed + 2)
    feats, _ = synthetic.point_attributes(n, channels, "normal", seed + 1)
    opac = rng.uniform(lo, hi, n).astype(np.float32)
    opac[::97] = 0.0
    if hi >= 1.0:
        opac[5::89] = 1.0
    run = H.GaussianRun(hv, pos, feats, opac, tile, channels).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, tile, channels)
    check_structure(run.debug(), ref)
    out = run.outputs()
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7 + 1e-6 * float(ref["blending_weights"].max()),
                   "blending weights")
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                               gaussian=g)
    H.assert_close(gf, gf_ref, RTOL, grad_atol(gf_ref), "feature gradients")
    H.assert_close(go, go_ref, RTOL, grad_atol(go_ref), "opacity gradients")
    # a second backward pass on the same saved state
    gf2, go2 = run.backward(gi, ga)
    # (instances without slots add with float atomics: the last bits depend on scheduling)
    H.assert_close(gf2, gf, RTOL, grad_atol(gf_ref), "feature gradients, second pass")
    H.assert_close(go2, go, RTOL, grad_atol(go_ref), "opacity gradients, second pass")
