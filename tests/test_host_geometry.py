"""The rasterizer's per-point arithmetic as the kernels run it (inpc_amd/csrc/geometry.hpp), compiled for the host by
tests/host_build and checked on the CPU, without a GPU: projection, tile bounds and depth keys bit for bit against the
oracle; footprint weights, fragment slots and gradient rows against independent restatements of the reference's blend
(B/rasterization/src/bilinear/kernels.cu:40-64,208-217,281-287); the Gaussian footprint's exponential against the
oracle's. The GPU tests check the same through the kernels; these hold the arithmetic itself where no GPU is at hand."""
from __future__ import annotations

import ctypes as C

import numpy as np
import pytest

from inpc_amd import _lib, synthetic
from tests.host_build import build as host_build


@pytest.fixture(scope="module")
def host():
    return host_build.lib()


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def project(host, hv, pos, tile):
    n = len(pos)
    cam = _lib.make_camera(hv.camera)
    out = {k: np.zeros(n, np.float32) for k in ("sx", "sy", "depth")}
    out.update({k: np.zeros(n, np.uint32) for k in ("info", "touched", "key")})
    pos = np.ascontiguousarray(pos, np.float32)
    w2c = np.ascontiguousarray(hv.w2c, np.float32)
    host.host_project(tile, C.byref(cam), _p(w2c), _p(pos), n, *(_p(out[k]) for k in ("sx", "sy", "depth", "info",
                                                                                     "touched", "key")))
    return out


def scene(n, seed, width=251, height=163, focal=230.0):
    hv = synthetic.rotated_camera(width, height, focal, 2.4, 0.2, -0.1)
    pos = synthetic.cube_points(n, 2.5, seed)     # wider than the frustum: many points are culled
    rng = np.random.default_rng(seed)
    pos[: n // 10, 2] -= 4.0                      # some behind the camera or in front of the near plane
    pos[n // 10: n // 5] *= rng.uniform(0.0, 0.05, (n // 5 - n // 10, 1)).astype(np.float32)
    return hv, pos


@pytest.mark.parametrize("tile", [8, 16])
def test_projection_bounds_and_keys_match_the_oracle(host, oracle, tile):
    n = 120000
    hv, pos = scene(n, 7 + tile)
    got = project(host, hv, pos, tile)
    c = hv.camera
    cam = oracle.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)
    cfg = oracle.make_config(n, cam, tile, 4, oracle.FEAT_DIRECT_F32)
    feats = np.zeros((n, 4), np.float32)
    ref = oracle.raster_forward(cfg, pos, feats, np.full(n, 0.5, np.float32), hv.w2c, debug=True)
    drawn = got["info"] != 0
    assert 0.2 * n < drawn.sum() < 0.9 * n and (ref["n_touched"] > 1).sum() > 1000
    np.testing.assert_array_equal(np.where(drawn, got["touched"], 0), ref["n_touched"])
    assert drawn.sum() == ref["n_visible"] and got["touched"][drawn].sum() == ref["n_instances"]
    xy = np.stack([got["sx"], got["sy"]], 1)
    np.testing.assert_array_equal(xy[drawn].view(np.uint32), ref["screen_xy"][drawn].view(np.uint32))
    np.testing.assert_array_equal(got["depth"][drawn].view(np.uint32), ref["depth"][drawn].view(np.uint32))
    gw = (c.width + tile - 1) // tile
    tile0 = got["info"] & 0xFFFF
    nx, ny = ((got["info"] >> 16) & 1) + 1, ((got["info"] >> 17) & 1) + 1
    bounds = np.stack([tile0 % gw, tile0 % gw + nx, tile0 // gw, tile0 // gw + ny], 1).astype(np.uint16)
    np.testing.assert_array_equal(bounds[drawn], ref["bounds"][drawn])
    assert (nx * ny == got["touched"])[drawn].all()
    # depth keys: the oracle lists the depths' float bits in depth order; the kernels sort on their offset from the
    # near plane's bits (the same order, fewer bits that differ)
    key_of_point = np.zeros(n, np.uint32)
    key_of_point[ref["depth_order"]] = ref["depth_keys"]
    bias = np.float32(c.near_plane).view(np.uint32)
    np.testing.assert_array_equal(got["key"][drawn] + bias, key_of_point[drawn])
    assert (np.diff(got["key"][ref["depth_order"]].astype(np.int64)) >= 0).all()
    assert (got["key"][~drawn] == 0xFFFFFFFF).all()


def reference_weights(s, pixel):
    """Interpolation weight of one axis as the reference's blend computes it per pixel (kernels.cu:284-287), fp32."""
    d = np.abs(np.float32(s) - (np.float32(pixel) + np.float32(0.5))).astype(np.float32)
    return np.where(d >= 1, np.float32(0), np.clip(np.float32(1) - d, np.float32(0), np.float32(1))).astype(np.float32)


def test_axis_weights_are_the_blends_per_pixel_weights(host):
    rng = np.random.default_rng(3)
    s = np.concatenate([rng.uniform(-3, 300, 200000), np.arange(-2, 40) + 0.5, np.arange(-2, 40).astype(np.float64),
                        np.arange(0, 40) + 0.5 - 2.0 ** -20, [-0.5, -0.4, 7.5, 8.0, 8.6, 65535.7, 1e9, -1e9]]).astype(np.float32)
    n = len(s)
    left, w0, w1 = np.zeros(n, np.int32), np.zeros(n, np.float32), np.zeros(n, np.float32)
    host.host_axis_weights(_p(s), n, _p(left), _p(w0), _p(w1))
    inside = (s > -0.5) & (s < 65000)
    expect_left = np.floor((s - np.float32(0.5)).astype(np.float32)).astype(np.int64)
    np.testing.assert_array_equal(left[inside], expect_left[inside])
    assert left.min() >= -1 and left.max() <= 65534
    np.testing.assert_array_equal(w0.view(np.uint32), reference_weights(s, left).view(np.uint32))
    np.testing.assert_array_equal(w1.view(np.uint32), reference_weights(s, left + 1).view(np.uint32))
    # no pixel but the two candidates can be closer than 1, and the two weights of an interior position add up to 1
    for other in (-1, 2):
        assert (reference_weights(s[inside], left[inside].astype(np.int64) + other) == 0).all()
    mid = inside & (s > 1) & (s < 60000)
    np.testing.assert_allclose(w0[mid] + w1[mid], 1.0, atol=2e-4)   # fp32 at coordinates up to a few hundred


@pytest.mark.parametrize("tile", [8, 16])
def test_fragment_slots_are_the_pixels_and_weights_of_the_reference_blend(host, tile):
    """Per tile a point's fragments: every pixel of the tile with |dx| < 1 and |dy| < 1 gets weight sat(1-dx) sat(1-dy)
    (kernels.cu:281-287). The kernels find them as four slots: for 16x16 tiles slot = parity class of the pixel (the wave
    that owns it), pixel = place in that wave's 8 x 8 grid; for 8x8 tiles slot = candidate pixel."""
    rng = np.random.default_rng(11 + tile)
    cases = [(float(sx), float(sy), int(tx) * tile, int(ty) * tile)
             for sx, sy, tx, ty in zip(rng.uniform(-1.5, 3 * tile + 1.5, 2500), rng.uniform(-1.5, 2 * tile + 1.5, 2500),
                                       rng.integers(0, 3, 2500), rng.integers(0, 2, 2500))]
    # positions on pixel centres, pixel borders and tile borders
    for v in (0.0, 0.5, 1.0, tile - 0.5, float(tile), tile + 0.5, 2.0 * tile, tile - 2.0 ** -18, tile + 2.0 ** -18):
        for t0 in (0, tile):
            cases += [(v, 5.25, t0, 0), (5.25, v, 0, t0), (v, v, t0, t0)]
    weight, pixel = np.zeros(4, np.float32), np.zeros(4, np.uint32)
    hits = 0
    for sx, sy, x0, y0 in cases:
        host.host_fragment_slots(tile, C.c_float(sx), C.c_float(sy), x0, y0, _p(weight), _p(pixel))
        got = {}
        for slot in range(4):
            if pixel[slot] == 0xFF:
                continue
            pix = int(pixel[slot])
            assert pix < 64
            if tile == 16:
                lx, ly = 2 * (pix & 7) + (slot & 1), 2 * (pix >> 3) + (slot >> 1)
            else:
                lx, ly = pix & 7, pix >> 3
            assert (lx, ly) not in got
            got[(lx, ly)] = weight[slot]
        expect = {}
        for ly in range(tile):
            for lx in range(tile):
                wx, wy = reference_weights(sx, x0 + lx), reference_weights(sy, y0 + ly)
                w = np.float32(wx * wy)
                if wx > 0 and wy > 0 and w > 0:
                    expect[(lx, ly)] = w
        assert got.keys() == expect.keys(), (sx, sy, x0, y0, got, expect)
        for k in got:
            assert np.float32(got[k]).view(np.uint32) == np.float32(expect[k]).view(np.uint32)
        hits += len(got)
    assert hits > 1000


@pytest.mark.parametrize("tile", [8, 16])
def test_gradient_rows_follow_the_order_the_instances_are_created_in(host, tile):
    """A point that touches several tiles gets one gradient row per tile, numbered in the row-major order of its tiles
    (kernels.cu:208-217); the forward blend of a tile works out its own row from the point's record alone."""
    n = 60000
    hv, pos = scene(n, 40 + tile, width=203, height=117)
    cam = _lib.make_camera(hv.camera)
    tiles, rows = np.zeros((n, 4), np.uint32), np.zeros((n, 4), np.uint32)
    pos = np.ascontiguousarray(pos, np.float32)
    w2c = np.ascontiguousarray(hv.w2c, np.float32)
    host.host_instance_rows(tile, C.byref(cam), _p(w2c), _p(pos), n, _p(tiles), _p(rows))
    got = project(host, hv, pos, tile)
    count = (tiles != 0xFFFFFFFF).sum(1)
    np.testing.assert_array_equal(count, got["touched"] * (got["info"] != 0))
    assert (count == 2).sum() > 500 and (count == 4).sum() > 50
    gw = (hv.camera.width + tile - 1) // tile
    for k in range(4):
        has = count > k
        np.testing.assert_array_equal(rows[has, k], 1000 + k)    # the k-th tile of a point has its k-th row
        if k:
            assert (tiles[has, k] > tiles[has, k - 1]).all()      # row-major: ascending tile ids
    # the tiles are the rectangle of the bounds
    four = count == 4
    assert (tiles[four, 1] == tiles[four, 0] + 1).all() and (tiles[four, 2] == tiles[four, 0] + gw).all()
    # points at the image's left and top rim, whose left / top candidate pixel lies outside the image: one tile less
    rim = (got["info"] != 0) & ((got["sx"] < 0.5) | (got["sy"] < 0.5))
    assert rim.sum() > 0 and (rows[rim, 0] == 1000).all()


def test_footprint_exp_is_the_oracles_bit_for_bit(host, oracle):
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.uniform(-30, 0, 20000), rng.uniform(-100, 5, 2000), -np.logspace(-8, 2, 500),
                        [0.0, -0.0, -87.0, -87.0001, -88.0, -1e30, np.nan, -np.inf, 1e-3]]).astype(np.float32)
    out = np.zeros_like(x)
    host.host_footprint_exp(_p(x), len(x), _p(out))
    ref = oracle.footprint_exp(x)
    np.testing.assert_array_equal(out.view(np.uint32), np.asarray(ref, np.float32).view(np.uint32))
    ok = (x <= 0) & (x >= -30)
    np.testing.assert_allclose(out[ok], np.exp(x[ok].astype(np.float64)), rtol=2e-7)


def test_footprint_value_cut(host):
    # exponent = -0.5 (a dx^2 + c dy^2) - b dx dy; a pixel is drawn when the exponent is not positive and the value
    # not below the threshold (B/rasterization/src/gaussian/kernels.cu:447-452)
    rng = np.random.default_rng(9)
    n = 5000
    cx = (rng.integers(0, 40, n) + 0.5).astype(np.float32)
    cy = (rng.integers(0, 40, n) + 0.5).astype(np.float32)
    G, drawn = np.zeros(n, np.float32), np.zeros(n, np.uint8)
    sx, sy, a, b, c_, thr = 20.3, 19.1, 0.21, 0.05, 0.33, 0.01110899653
    host.host_footprint_value(C.c_float(sx), C.c_float(sy), C.c_float(a), C.c_float(b), C.c_float(c_), C.c_float(thr),
                              _p(cx), _p(cy), n, _p(G), _p(drawn))
    dx, dy = np.float64(np.float32(sx)) - cx, np.float64(np.float32(sy)) - cy
    exact = np.exp(-0.5 * (np.float32(a) * dx * dx + np.float32(c_) * dy * dy) - np.float32(b) * dx * dy)
    clear = np.abs(exact - thr) > 1e-5
    np.testing.assert_array_equal(drawn[clear].astype(bool), exact[clear] >= thr)
    np.testing.assert_allclose(G[drawn.astype(bool)], exact[drawn.astype(bool)], rtol=3e-6)
    assert 50 < drawn.sum() < n - 50
