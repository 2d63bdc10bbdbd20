"""The benchmark configurations at their real sizes, through the C ABI, against the CPU oracle on the same inputs
(the oracle finishes each of them in seconds to tens of seconds on the host cores), plus size-independent
properties: every drawn sample lies in the frustum and in its leaf, the depth order is sorted, tile ranges
partition the instance list, blending weights are consistent with the image alpha.

Bit-exact: sample ids and positions, generator state, tile bounds, keys, sort orders, tile ranges.
Within 1e-4 relative plus a small absolute floor: images, blending weights, gradients.
"""
import numpy as np
import pytest
import torch

from inpc_amd import ProbabilityFieldSampler, _lib, synthetic
from tests import helpers as H
from tests.test_gpu_raster import check_structure, oracle_cfg

pytestmark = pytest.mark.gpu

RTOL = 1e-4


def oracle_cam(O, hv):
    c = hv.camera
    return O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)


def test_config0_small_forward(gpu, oracle):
    """65,536 uniform points in the unit cube, 4 direct fp32 channels, 256x256, f = 300, distance 3, 16x16 tiles."""
    n = 65536
    hv = synthetic.camera_on_z(256, 256, 300.0, 3.0)
    pos = synthetic.cube_points(n, 1.0, 0)
    feats, opac = synthetic.point_attributes(n, 4, "uniform", 0)
    run = H.RasterRun(hv, pos, feats, opac, 16, 4, _lib.FEAT_DIRECT_F32).forward()
    ref = oracle.raster_forward(oracle_cfg(oracle, hv, n, 16, 4, oracle.FEAT_DIRECT_F32), pos, feats, opac, hv.w2c,
                                debug=True)
    check_structure(run.debug(), ref)
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 1e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")


@pytest.fixture(scope="module")
def config1(gpu, oracle):
    """262,144 leaves of the level-9 grid over [-2,2]^3, camera 1237x822 f = 1000 at (0,0,-6); 8,388,608 training
    samples drawn on the GPU and by the oracle."""
    n = 8_388_608
    oct = synthetic.octree_leaves(262_144, 9, 4.0, seed=0)
    hv = synthetic.camera_on_z(1237, 822, 1000.0, 6.0)
    view = hv.to_view(gpu)
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    sampler = ProbabilityFieldSampler(seed=0)
    pos, ids = sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
    rng_ref = oracle.Pcg32(0)
    pos_ref, ids_ref, consumed = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c,
                                                         oracle_cam(oracle, hv), oct.initial_size, rng_ref, n)
    return dict(n=n, oct=oct, hv=hv, sampler=sampler, pos=pos, ids=ids, pos_ref=pos_ref, ids_ref=ids_ref,
                consumed=consumed, rng_ref=rng_ref)


def test_config1_training_draw_bit_exact(config1, oracle):
    c = config1
    ids = c["ids"].cpu().numpy()
    pos = c["pos"].cpu().numpy()
    np.testing.assert_array_equal(ids, c["ids_ref"].astype(np.int64))
    np.testing.assert_array_equal(pos.view(np.uint32), c["pos_ref"].view(np.uint32))
    assert c["sampler"].last_consumed == c["consumed"] > c["n"]   # the view culls some candidates
    assert c["sampler"].rng_state() == (int(c["rng_ref"].state[0]), int(c["rng_ref"].state[1]))


def test_config1_sample_properties(config1):
    c = config1
    oct, hv = c["oct"], c["hv"]
    ids = c["ids"].cpu().numpy()
    pos = c["pos"].cpu().numpy()
    assert ids.min() >= 0 and ids.max() < len(oct.weights)
    half = oct.initial_size / 2.0 ** (oct.levels[ids].astype(np.float64) + 1)
    assert (np.abs(pos.astype(np.float64) - oct.centers[ids]) <= half[:, None] * (1 + 1e-6)).all()
    m = hv.w2c.astype(np.float64)
    q = pos.astype(np.float64) @ m[:3, :3].T + m[:3, 3]
    cam = hv.camera
    x = q[:, 0] / q[:, 2] * cam.focal_x + cam.center_x
    y = q[:, 1] / q[:, 2] * cam.focal_y + cam.center_y
    eps = 1e-3
    assert ((q[:, 2] >= cam.near_plane) & (q[:, 2] <= cam.far_plane)).all()
    assert ((x > -eps) & (x < cam.width + eps) & (y > -eps) & (y < cam.height + eps)).all()
    # leaf frequencies follow the view-dependent weights: compare the 64 heaviest leaves with their expectation
    counts = np.bincount(ids, minlength=len(oct.weights)).astype(np.float64)
    top = np.argsort(counts)[-64:]
    assert counts[top].min() > 500
    # ratio of counts between leaves at the same level and (nearly) the same depth equals the ratio of weights
    depth = oct.centers[top].astype(np.float64) @ m[2, :3] + m[2, 3]
    expect = oct.weights[top].astype(np.float64) / np.maximum(np.abs(depth - cam.near_plane) / cam.far_plane, 1e-8)
    ratio = (counts[top] / counts[top].sum()) / (expect / expect.sum())
    assert np.abs(ratio - 1).max() < 0.2


@pytest.mark.parametrize("tile", [16, 8])
def test_config2_and_3_forward_backward_full_size(config1, oracle, tile):
    """Config 2 (forward) and 3 (forward + backward): the 8,388,608 drawn points, 8 fp32 channels ~N(0,1),
    opacity = sigmoid(N(0,1)), gradients ~N(0,1e-2)."""
    c = config1
    n, hv = c["n"], c["hv"]
    pos = c["pos_ref"]
    feats, opac = synthetic.point_attributes(n, 8, "normal", 1)
    run = H.RasterRun(hv, pos, feats, opac, tile, 8, _lib.FEAT_DIRECT_F32).forward()
    cfg = oracle_cfg(oracle, hv, n, tile, 8, oracle.FEAT_DIRECT_F32)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    dbg = run.debug()
    check_structure(dbg, ref)
    # size-independent structure: depth keys ascend inside every tile's list, ranges partition the instance list in
    # tile order
    same_tile = np.diff(dbg["instance_keys"].astype(np.int64)) == 0
    assert (np.diff(dbg["instance_depth_keys"].astype(np.int64))[same_tile] >= 0).all()
    assert (np.diff(dbg["instance_keys"].astype(np.int64)) >= 0).all()
    r = dbg["tile_ranges"].astype(np.int64)
    used = r[:, 1] > r[:, 0]
    assert (r[used, 1] - r[used, 0]).sum() == dbg["n_instances"]
    assert (r[used][1:, 0] == r[used][:-1, 1]).all() and r[used][0, 0] == 0 and r[used][-1, 1] == dbg["n_instances"]
    del dbg
    out = run.outputs()
    H.assert_close(out["image"], ref["image"], RTOL, 2e-5, "image")
    H.assert_close(out["alpha"], ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    assert np.isfinite(out["image"]).all() and out["alpha"].min() >= 0 and out["alpha"].max() <= 1
    rng = np.random.default_rng(3)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
    H.assert_close(gf, gf_ref, RTOL, 2e-7, "feature gradients")
    H.assert_close(go, go_ref, RTOL, 2e-6, "opacity gradients")
    # linearity of the backward in the upstream gradient: doubling it doubles the result exactly (powers of two)
    gf2, go2 = run.backward(2 * gi, 2 * ga)
    H.assert_close(gf2, 2 * gf, 1e-5, 1e-9, "feature gradients, doubled input")
    H.assert_close(go2, 2 * go, 1e-5, 1e-8, "opacity gradients, doubled input")


def test_config3_points_gaussian_footprint_full_size(config1, oracle):
    """The 8,388,608 points of config 3 through the Gaussian footprint (training variance), 8x8 tiles, forward and
    backward, against the oracle: structure, image and alpha bit-exact, weights and gradients to tolerance."""
    from tests.test_gpu_gaussian import check_structure as check_gaussian_structure, grad_atol, oracle_run

    c = config1
    n, hv = c["n"], c["hv"]
    pos = c["pos_ref"]
    feats, opac = synthetic.point_attributes(n, 8, "normal", 1)
    run = H.GaussianRun(hv, pos, feats, opac, 8, 8).forward()
    g, ref = oracle_run(oracle, hv, pos, feats, opac, 8, 8)
    dbg = run.debug()
    check_gaussian_structure(dbg, ref)
    assert (np.diff(dbg["instance_keys"].astype(np.int64)) >= 0).all()
    r = dbg["tile_ranges"].astype(np.int64)
    used = r[:, 1] > r[:, 0]
    assert (r[used, 1] - r[used, 0]).sum() == dbg["n_instances"]
    del dbg
    out = run.outputs()
    np.testing.assert_array_equal(out["image"].view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(out["alpha"].view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, "blending weights")
    rng = np.random.default_rng(3)
    gi = rng.normal(0, 1e-2, ref["image"].shape).astype(np.float32)
    ga = rng.normal(0, 1e-2, ref["alpha"].shape).astype(np.float32)
    gf, go = run.backward(gi, ga)
    gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                               gaussian=g)
    H.assert_close(gf, gf_ref, RTOL, grad_atol(gf_ref), "feature gradients")
    H.assert_close(go, go_ref, RTOL, grad_atol(go_ref), "opacity gradients")
    # the gradient sums have a fixed order: a second backward gives the same bits
    gf2, go2 = run.backward(gi, ga)
    np.testing.assert_array_equal(gf2.view(np.uint32), gf.view(np.uint32))
    np.testing.assert_array_equal(go2.view(np.uint32), go.view(np.uint32))


@pytest.mark.real_gpu   # 33,554,432 points: hours in the simulator
def test_config4_large_frame_inference(gpu, oracle):
    """2,097,152 leaves of the level-11 grid, 33,554,432 samples, 16 channels stored as fp16, 2473x1643, f = 2000,
    16x16 tiles: sampling + inference forward end to end."""
    n = 33_554_432
    oct = synthetic.octree_leaves(2_097_152, 11, 4.0, seed=0)
    hv = synthetic.camera_on_z(2473, 1643, 2000.0, 6.0)
    view = hv.to_view(gpu)
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    sampler = ProbabilityFieldSampler(seed=0)
    pos_dev, ids_dev = sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
    rng_ref = oracle.Pcg32(0)
    pos_ref, ids_ref, consumed = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c,
                                                         oracle_cam(oracle, hv), oct.initial_size, rng_ref, n)
    np.testing.assert_array_equal(ids_dev.cpu().numpy(), ids_ref.astype(np.int64))
    pos = pos_dev.cpu().numpy()
    np.testing.assert_array_equal(pos.view(np.uint32), pos_ref.view(np.uint32))
    assert sampler.last_consumed == consumed
    del ids_dev, ids_ref, pos_ref
    gen = torch.Generator(device=gpu).manual_seed(4)
    feats_dev = torch.randn((n, 16), generator=gen, device=gpu, dtype=torch.float32).half()
    opac_dev = torch.sigmoid(torch.randn(n, generator=gen, device=gpu, dtype=torch.float32))
    feats, opac = feats_dev.cpu().numpy(), opac_dev.cpu().numpy()
    from inpc_amd.rasterization import rasterize_points

    image, depth, alpha = rasterize_points(view, pos_dev, feats_dev, opac_dev, tile=16, inference=True)
    torch.cuda.synchronize()
    cfg = oracle_cfg(oracle, hv, n, 16, 16, oracle.FEAT_DIRECT_F16, inference=True)
    ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c)
    H.assert_close(image.cpu().numpy(), ref["image"], RTOL, 2e-5, "image")
    H.assert_close(alpha.cpu().numpy(), ref["alpha"], RTOL, 1e-6, "alpha")
    H.assert_close(depth.cpu().numpy(), ref["depth_image"], RTOL, 1e-5, "depth")
    del image, depth, alpha, ref

    # the same 33,554,432 points through the Gaussian footprint's inference variant (sigma_world 0.002, cut at 3 sigma),
    # 8x8 tiles: 63,860 tiles, close to the limit of the 16-bit tile key
    from tests.test_oracle_gaussian import gcfg_of

    kw = dict(sigma_world=0.002, sigma_cutoff=3.0)
    image, depth, alpha = rasterize_points(view, pos_dev, feats_dev, opac_dev, tile=8, inference=True, mode=1, **kw)
    torch.cuda.synchronize()
    g = gcfg_of(oracle, hv, n, 8, 16, oracle.FEAT_DIRECT_F16, inference=True, **kw)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, gaussian=g)
    np.testing.assert_array_equal(image.cpu().numpy().view(np.uint32), ref["image"].view(np.uint32))
    np.testing.assert_array_equal(alpha.cpu().numpy().view(np.uint32), ref["alpha"].view(np.uint32))
    H.assert_close(depth.cpu().numpy(), ref["depth_image"], RTOL, 1e-5, "Gaussian footprint depth")
