"""Pins the oracle's Gaussian footprint (B/rasterization/src/gaussian/kernels.cu) against float64 closed forms,
numpy's sorts and a float64 brute-force blend with central differences for the gradients (CPU only).

The reference holds no test or fixture for this mode; what the mathematics fixes is checked here: the exponential,
the covariance / conic / tile bounds, the instance order, the blend (image, alpha, depth, blending weights with the
extra footprint factor) and the gradients."""
import numpy as np
import pytest

from inpc_amd import synthetic
from test_oracle_raster import cam_of, project64

TRAIN_THRESHOLD = 0.01110899653


def gcfg_of(O, hv, n, tile, channels, mode=None, inference=False, sigma_world=0.0, sigma_cutoff=3.0):
    mode = O.FEAT_DIRECT_F32 if mode is None else mode
    base = O.make_config(n, cam_of(O, hv), tile, channels, mode, O.RASTER_INFERENCE if inference else 0)
    return O.GaussianConfig(base, sigma_world, sigma_cutoff, 0, 0)


def covariance64(hv, pos, variance):
    """cov2d of kernels.cu:57-72 in float64: returns sx, sy, depth, cov (n,3), conic (n,3)."""
    c = hv.camera
    m = hv.w2c.astype(np.float64)
    q = pos.astype(np.float64) @ m[:3, :3].T + m[:3, 3]
    z = q[:, 2]
    x, y = q[:, 0] / z, q[:, 1] / z
    j00, j11 = c.focal_x / z, c.focal_y / z
    lx, ly = 1.3 * c.center_x / c.focal_x, 1.3 * c.center_y / c.focal_y
    j02 = -j00 * np.clip(x, -lx, lx)
    j12 = -j11 * np.clip(y, -ly, ly)
    variance = np.broadcast_to(np.asarray(variance, np.float64), z.shape)
    cov = np.stack([variance * (j00 * j00 + j02 * j02) + 0.16, variance * (j02 * j12),
                    variance * (j11 * j11 + j12 * j12) + 0.16], 1)
    det = cov[:, 0] * cov[:, 2] - cov[:, 1] ** 2
    conic = np.stack([cov[:, 2] / det, -cov[:, 1] / det, cov[:, 0] / det], 1)
    return x * c.focal_x + c.center_x, y * c.focal_y + c.center_y, z, cov, conic


def near_camera_points(hv, n, seed):
    """Points 0.012 to 0.06 in front of the camera, inside the image: footprints of 3 to 13 pixels sigma."""
    rng = np.random.default_rng(seed)
    c = hv.camera
    depth = 0.012 + 0.048 * rng.random(n)
    u = (rng.random(n) - 0.5) * c.width / c.focal_x * depth
    v = (rng.random(n) - 0.5) * c.height / c.focal_y * depth
    r = hv.w2c[:3, :3].astype(np.float64)
    cam_space = np.stack([u, v, depth], 1)
    return ((cam_space - hv.w2c[:3, 3].astype(np.float64)) @ r).astype(np.float32)   # R^T (q - t)


def brute_force(hv, sx, sy, z, conic, bounds, touched, feats, opac, order, tile, threshold):
    """Per pixel, front to back over all drawn points in the given order; a point reaches a pixel when the pixel's
    tile lies inside the point's tile bounds and the footprint passes the threshold (kernels.cu:401-474)."""
    c = hv.camera
    C_ = feats.shape[1]
    img = np.zeros((C_, c.height, c.width))
    dep = np.zeros((c.height, c.width))
    Tr = np.ones((c.height, c.width))
    done = np.zeros((c.height, c.width), bool)
    bw_out = np.zeros(len(sx))
    f64 = feats.astype(np.float64)
    for i in order:
        if not touched[i]:
            continue
        x0, x1, y0, y1 = [int(v) for v in bounds[i]]
        for py in range(y0 * tile, min(y1 * tile, c.height)):
            for px in range(x0 * tile, min(x1 * tile, c.width)):
                if done[py, px]:
                    continue
                dx, dy = sx[i] - (px + 0.5), sy[i] - (py + 0.5)
                e = -0.5 * (conic[i, 0] * dx * dx + conic[i, 2] * dy * dy) - conic[i, 1] * dx * dy
                if e > 0:
                    continue
                G = np.exp(e)
                if G < threshold:
                    continue
                a = float(opac[i]) * G
                b = Tr[py, px] * a
                if b > 0:
                    bw_out[i] += G * b
                img[:, py, px] += b * f64[i]
                dep[py, px] += b * z[i]
                Tr[py, px] *= 1 - a
                if Tr[py, px] < 1e-4:
                    done[py, px] = True
    alpha = np.where(Tr < 1e-4, 1.0, 1 - Tr)
    depth_img = np.where(1 - Tr > 0, dep / np.maximum(1 - Tr, 1e-300), 0.0)
    return img, alpha, bw_out, depth_img


def test_footprint_exp_is_exp_to_one_ulp(oracle):
    rng = np.random.default_rng(0)
    x = -(rng.random(100000) * 30).astype(np.float32)
    x[:6] = [0.0, -4.5, -0.5, -87.0, -1e-8, -20.0]
    got = oracle.footprint_exp(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - want) / ulp) < 1.5
    assert got[0] == 1.0
    assert oracle.footprint_exp(np.float32(-88.0)) == 0.0 and oracle.footprint_exp(np.float32(-1e30)) == 0.0
    # monotone: the cut at a threshold is a cut at a radius
    xs = np.sort(x)
    assert np.all(np.diff(oracle.footprint_exp(xs)) >= 0)


@pytest.mark.parametrize("tile", [8, 16])
def test_covariance_conic_and_bounds_against_float64(oracle, tile):
    n = 20000
    hv = synthetic.rotated_camera(150, 97, 120.0, 2.5, 0.3, 0.2)
    pos = synthetic.cube_points(n, 1.8, 3)
    pos[:500] = near_camera_points(hv, 500, 9)   # large footprints, many tiles
    feats, opac = synthetic.point_attributes(n, 4, "uniform", 4)
    g = gcfg_of(oracle, hv, n, tile, 4)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    c = hv.camera
    variance = (0.3 * 0.5) ** 2 / (c.focal_x * c.focal_y)
    sx, sy, z, cov, conic = covariance64(hv, pos, variance)
    vis = ref["n_touched"] > 0
    assert vis.sum() > n // 2
    np.testing.assert_allclose(ref["conic"][vis], conic[vis], rtol=2e-4, atol=2e-6)
    # tile bounds: floor / ceil of (s -+ (3 sigma - 0.5)) / T, clamped to the grid; compared where float64 is not
    # within rounding of a tile edge
    gw, gh = (c.width + tile - 1) // tile, (c.height + tile - 1) // tile
    rx, ry = 3 * np.sqrt(cov[:, 0]) - 0.5, 3 * np.sqrt(cov[:, 2]) - 0.5
    raw = np.stack([(sx - rx) / tile, (sx + rx) / tile, (sy - ry) / tile, (sy + ry) / tile], 1)
    want = np.stack([np.clip(np.floor(raw[:, 0]), 0, gw), np.clip(np.ceil(raw[:, 1]), 0, gw),
                     np.clip(np.floor(raw[:, 2]), 0, gh), np.clip(np.ceil(raw[:, 3]), 0, gh)], 1)
    inside = (z >= c.near_plane) & (z <= c.far_plane)
    touched = np.where(inside, (want[:, 1] - want[:, 0]) * (want[:, 3] - want[:, 2]), 0)
    safe = np.all(np.abs(raw - np.round(raw)) > 1e-4, axis=1)
    np.testing.assert_array_equal(ref["n_touched"][safe], touched[safe].astype(np.uint32))
    both = safe & vis
    np.testing.assert_array_equal(ref["bounds"][both], want[both].astype(np.uint16))
    assert ref["n_touched"].max() > 4        # the footprint is not limited to 2 x 2 tiles
    assert ref["n_instances"] == ref["n_touched"].sum() == count


def test_instance_order_against_numpy_sorts(oracle):
    n, tile = 6000, 8
    hv = synthetic.rotated_camera(150, 97, 120.0, 2.5, 0.3, 0.2)
    pos = synthetic.cube_points(n, 1.8, 5)
    pos[:300] = pos[300:600]       # equal depth keys fall back to the point id
    feats, opac = synthetic.point_attributes(n, 4, "uniform", 6)
    g = gcfg_of(oracle, hv, n, tile, 4)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    gw = (150 + tile - 1) // tile
    vis = np.flatnonzero(ref["n_touched"])
    keys = ref["depth"].view(np.uint32)[vis]
    order = vis[np.lexsort((vis, keys))]
    np.testing.assert_array_equal(ref["depth_order"], order)
    b = ref["bounds"].astype(np.int64)
    rank = np.empty(n, np.int64)
    rank[order] = np.arange(len(order))
    inst_tile, inst_point = [], []
    for i in vis:
        for ty in range(b[i, 2], b[i, 3]):
            for tx in range(b[i, 0], b[i, 1]):
                inst_tile.append(ty * gw + tx)
                inst_point.append(i)
    inst_tile, inst_point = np.array(inst_tile), np.array(inst_point)
    final = np.lexsort((rank[inst_point], inst_tile))
    np.testing.assert_array_equal(ref["instance_keys"], inst_tile[final].astype(np.uint16))
    np.testing.assert_array_equal(ref["instance_points"], inst_point[final].astype(np.uint32))
    ranges = ref["tile_ranges"]
    for t in np.unique(inst_tile):
        where = np.flatnonzero(inst_tile[final] == t)
        assert tuple(ranges[t]) == (where[0], where[-1] + 1)


def small_scene(seed, n=700, layered=False):
    hv = synthetic.rotated_camera(48, 37, 40.0, 2.5, 0.25, -0.15)
    pos = synthetic.cube_points(n, 1.6, seed)
    feats, opac = synthetic.point_attributes(n, 4, "uniform", seed + 1)
    if layered:   # twelve spots with forty nearly opaque points each: many layers per pixel, early termination
        for k in range(12):
            pos[40 * k: 40 * (k + 1)] = pos[600 + k]
        opac[:480] = 0.97
    return hv, pos, feats, opac


@pytest.mark.parametrize("tile", [8, 16])
def test_training_blend_against_float64_brute_force(oracle, tile):
    hv, pos, feats, opac = small_scene(11, layered=True)
    n = len(pos)
    g = gcfg_of(oracle, hv, n, tile, 4)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    # geometry as the oracle rounded it (pinned by the tests above); the blend in float64
    sx, sy = ref["screen_xy"][:, 0].astype(np.float64), ref["screen_xy"][:, 1].astype(np.float64)
    img, alpha, bw, _ = brute_force(hv, sx, sy, ref["depth"].astype(np.float64), ref["conic"].astype(np.float64),
                                    ref["bounds"], ref["n_touched"], feats, opac, ref["depth_order"], tile, TRAIN_THRESHOLD)
    assert (alpha == 1.0).sum() > 10, "the scene must exercise early termination"
    np.testing.assert_allclose(ref["image"], img, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(ref["alpha"][0], alpha, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(ref["blending_weights"], bw, rtol=2e-4, atol=2e-5)


def test_single_point_known_answer(oracle):
    # identity camera, focal 1000, a point on the axis at depth 50: the footprint is the dilation alone up to 1e-7,
    # cov = 0.16 I, conic = 6.25 I: centre pixel G = exp(-0.5 * 6.25 * (0.5^2 + 0.5^2)); 3 sigma = 1.2 pixels
    from inpc_amd.views import PerspectiveCamera

    cam = PerspectiveCamera(32, 32, 1000.0, 1000.0, 16.0, 16.0, 0.01, 100.0)
    hv = synthetic.HostView(cam, np.eye(4, dtype=np.float32), np.zeros(3, np.float32))
    pos = np.array([[0.0, 0.0, 50.0]], np.float32)   # projects to (16, 16): the corner of four pixels
    feats = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    opac = np.array([0.5], np.float32)
    g = gcfg_of(oracle, hv, 1, 8, 4)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=64)
    np.testing.assert_allclose(ref["conic"][0], [6.25, 0.0, 6.25], rtol=1e-4, atol=1e-6)
    assert ref["n_touched"][0] == 4 and list(ref["bounds"][0]) == [1, 3, 1, 3]   # 16 -+ 0.7 -> tiles 1 and 2
    G_near = np.exp(-0.5 * 6.25 * 0.5)            # the four pixels around the point: d = (0.5, 0.5)
    G_far = np.exp(-0.5 * 6.25 * (0.25 + 2.25))   # d = (0.5, 1.5): 4e-4, below the threshold
    assert G_far < TRAIN_THRESHOLD < G_near
    want = np.zeros((32, 32))
    want[15:17, 15:17] = 0.5 * G_near
    np.testing.assert_allclose(ref["alpha"][0], want, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(ref["image"][2], 3.0 * want, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(ref["blending_weights"][0], 4 * G_near * 0.5 * G_near, rtol=5e-4)


@pytest.mark.parametrize("with_scales", [False, True])
def test_inference_blend_against_float64_brute_force(oracle, with_scales):
    hv, pos, feats, opac = small_scene(21)
    n, tile = len(pos), 8
    sigma_world, cutoff = 0.004, 2.5
    scales = (np.random.default_rng(5).random(n) * 0.008).astype(np.float32) if with_scales else None
    g = gcfg_of(oracle, hv, n, tile, 4, inference=True, sigma_world=sigma_world, sigma_cutoff=cutoff)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c, scales)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, scales=scales,
                                n_instances_hint=count)
    variance = scales.astype(np.float64) ** 2 if with_scales else float(np.float32(sigma_world)) ** 2
    sx, sy, z, cov, conic = covariance64(hv, pos, variance)
    vis = ref["n_touched"] > 0
    np.testing.assert_allclose(ref["conic"][vis], conic[vis], rtol=2e-4, atol=2e-6)
    # bounds reach cutoff * sigma - 0.5
    rx = cutoff * np.sqrt(cov[:, 0]) - 0.5
    raw = (sx - rx) / tile
    safe = vis & (np.abs(raw - np.round(raw)) > 1e-4)
    np.testing.assert_array_equal(ref["bounds"][safe, 0], np.clip(np.floor(raw[safe]), 0, 6).astype(np.uint16))
    threshold = np.exp(-0.5 * cutoff * cutoff)
    img, alpha, _, depth = brute_force(hv, ref["screen_xy"][:, 0].astype(np.float64), ref["screen_xy"][:, 1].astype(np.float64),
                                       ref["depth"].astype(np.float64), ref["conic"].astype(np.float64), ref["bounds"],
                                       ref["n_touched"], feats, opac, ref["depth_order"], tile, threshold)
    np.testing.assert_allclose(ref["image"], img, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(ref["alpha"][0], alpha, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(ref["depth_image"][0], depth, rtol=2e-4, atol=2e-5)
    assert ref["blending_weights"] is None


def test_backward_against_central_differences(oracle):
    hv, pos, feats, opac = small_scene(31, n=260)
    opac = (0.1 + 0.6 * opac).astype(np.float32)    # no pixel saturates: the loss is smooth in features and opacities
    n, tile = len(pos), 8
    g = gcfg_of(oracle, hv, n, tile, 4)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    assert ref["alpha"].max() < 0.999
    rng = np.random.default_rng(3)
    gi = rng.standard_normal(ref["image"].shape).astype(np.float32)
    ga = rng.standard_normal(ref["alpha"].shape).astype(np.float32)
    gf, go, gv = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c, gaussian=g)
    np.testing.assert_array_equal(gf, gv)
    geom = (ref["screen_xy"][:, 0].astype(np.float64), ref["screen_xy"][:, 1].astype(np.float64),
            ref["depth"].astype(np.float64), ref["conic"].astype(np.float64), ref["bounds"], ref["n_touched"])

    def loss(f, o):
        img, alpha, _, _ = brute_force(hv, *geom, f, o, ref["depth_order"], tile, TRAIN_THRESHOLD)
        return float((img * gi).sum() + (alpha * ga[0]).sum())

    drawn = np.flatnonzero(ref["blending_weights"] > 1e-3)
    assert len(drawn) > 20
    eps = 1e-5
    for i in drawn[:: max(1, len(drawn) // 12)]:
        o_hi, o_lo = opac.astype(np.float64), opac.astype(np.float64)
        o_hi[i] += eps
        o_lo[i] -= eps
        d = (loss(feats.astype(np.float64), o_hi) - loss(feats.astype(np.float64), o_lo)) / (2 * eps)
        np.testing.assert_allclose(go[i], d, rtol=2e-3, atol=2e-4)
        for ch in (0, 3):
            f_hi, f_lo = feats.astype(np.float64), feats.astype(np.float64)
            f_hi[i, ch] += eps
            f_lo[i, ch] -= eps
            d = (loss(f_hi, opac.astype(np.float64)) - loss(f_lo, opac.astype(np.float64))) / (2 * eps)
            np.testing.assert_allclose(gf[i, ch], d, rtol=2e-3, atol=2e-4)
    # points that are not drawn get exact zeros
    hidden = ref["n_touched"] == 0
    assert np.all(gf[hidden] == 0) and np.all(go[hidden] == 0)
    # the audit outputs the GPU tests judge gradients by (pinned against autograd for the bilinear footprint, whose
    # code they share): the same derivatives, sums of magnitudes that bound the sums, zeros for hidden points, and the
    # fp32 sums within the bound the GPU results are held to
    from tests import helpers as H
    gf2, go2, _, audit = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c,
                                                gaussian=g, audit=True)
    # (two runs of the oracle differ in the last bits where a point lies in several tiles: its threads add in turn)
    np.testing.assert_allclose(gf2, gf, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(go2, go, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(audit["view64"], gf, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(audit["opacity64"], go, rtol=1e-4, atol=1e-4)
    assert (audit["view_abs"] >= np.abs(audit["view64"]) * (1 - 1e-12)).all()
    assert (audit["opacity_abs"] >= np.abs(audit["opacity64"]) * (1 - 1e-12)).all()
    assert np.all(audit["view_abs"][hidden] == 0) and np.all(audit["opacity_abs"][hidden] == 0)
    H.assert_gradient_close(gf, audit, "view", "fp32 feature gradients")
    H.assert_gradient_close(go, audit, "opacity", "fp32 opacity gradients")


def test_backward_on_saturating_pixels(oracle):
    # The branch the smooth scene above never takes: pixels whose transmittance falls below 1e-4. The fragment that
    # crosses the threshold still gets its gradient, the ones behind it get none
    # (B/rasterization/src/gaussian/kernels.cu:476-579); the brute force ends a pixel's list the same way, so its
    # central differences are those of the truncated blend.
    hv, pos, feats, opac = small_scene(41, n=1100)
    for k in range(60):   # sixty spots with sixteen nearly opaque points each
        pos[16 * k: 16 * (k + 1)] = pos[1000 + k]
    opac[:960] = 0.97
    n, tile = len(pos), 8
    g = gcfg_of(oracle, hv, n, tile, 4)
    count = oracle.gaussian_instance_count(g, pos, hv.w2c)
    ref = oracle.raster_forward(g.base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    saturated = ref["alpha"][0] == 1.0
    assert saturated.sum() >= 40, "the scene must saturate many pixels"
    rng = np.random.default_rng(5)
    gi = rng.standard_normal(ref["image"].shape).astype(np.float32)
    ga = rng.standard_normal(ref["alpha"].shape).astype(np.float32)
    gf, go, _ = oracle.raster_backward(g.base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c, gaussian=g)
    assert np.isfinite(gf).all() and np.isfinite(go).all()
    geom = (ref["screen_xy"][:, 0].astype(np.float64), ref["screen_xy"][:, 1].astype(np.float64),
            ref["depth"].astype(np.float64), ref["conic"].astype(np.float64), ref["bounds"], ref["n_touched"])

    def loss(f, o):
        img, alpha, _, _ = brute_force(hv, *geom, f, o, ref["depth_order"], tile, TRAIN_THRESHOLD)
        return float((img * gi).sum() + (alpha * ga[0]).sum())

    # The sixteen points of a spot coincide, so they are drawn in index order: the first ones are reached on every
    # pixel of their footprint, the last ones lie behind the cut on the spot's saturated centre pixel and are only
    # reached on the pixels around it. Both kinds must have the truncated blend's derivative.
    _, alpha_bf, _, _ = brute_force(hv, *geom, feats, opac, ref["depth_order"], tile, TRAIN_THRESHOLD)
    np.testing.assert_array_equal(alpha_bf == 1.0, saturated)
    spots = [k for k in range(60) if ref["n_touched"][16 * k] > 0]
    reached = np.array([16 * k + j for k in spots[::6] for j in (0, 15)])
    assert len(reached) >= 10
    eps = 1e-6
    for i in reached:
        o_hi, o_lo = opac.astype(np.float64), opac.astype(np.float64)
        o_hi[i] += eps
        o_lo[i] -= eps
        d = (loss(feats.astype(np.float64), o_hi) - loss(feats.astype(np.float64), o_lo)) / (2 * eps)
        np.testing.assert_allclose(go[i], d, rtol=5e-3, atol=5e-4)
        f_hi, f_lo = feats.astype(np.float64), feats.astype(np.float64)
        f_hi[i, 1] += 1e-4
        f_lo[i, 1] -= 1e-4
        d = (loss(f_hi, opac.astype(np.float64)) - loss(f_lo, opac.astype(np.float64))) / 2e-4
        np.testing.assert_allclose(gf[i, 1], d, rtol=2e-3, atol=2e-4)
