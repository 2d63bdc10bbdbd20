"""The committed fixtures of tests/golden (written by tests/golden/make_golden.py from the CPU oracle on three small
seeded cases): the oracle must still give them, and the HIP path must give them through the C ABI.

Bit-exact: leaf weights, CDF, sample ids and positions, generator states, tile bounds, screen coordinates, depth
keys and order, instances, tile ranges. Within 1e-4 relative: image, alpha, blending weights, gradients."""
import importlib.util
from pathlib import Path

import numpy as np
import pytest

GOLDEN = Path(__file__).resolve().parent / "golden"
RTOL = 1e-4


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a


EXACT_SAMPLER = ("leaf_weights", "cdf", "total", "plain_positions", "plain_ids", "plain_state", "training_positions",
                 "training_ids", "training_consumed", "training_state")
EXACT_RASTER = ("n_visible", "n_instances", "n_touched", "bounds", "screen_xy", "depth_keys", "depth_order",
                "instance_keys", "instance_points", "tile_ranges")
CLOSE_RASTER = {"image": 1e-5, "alpha": 1e-6, "blending_weights": 1e-7, "grad_features": 1e-7, "grad_opacities": 2e-7}


def test_oracle_reproduces_sampler_fixture(oracle, maker):
    want = np.load(GOLDEN / "sampler_small.npz")
    got = maker.sampler_answers()
    for key in EXACT_SAMPLER:
        np.testing.assert_array_equal(_bits(np.asarray(got[key])), _bits(want[key]), err_msg=key)


def test_oracle_reproduces_raster_fixture(oracle, maker):
    want = np.load(GOLDEN / "raster_small.npz")
    got = maker.raster_answers()
    for key in EXACT_RASTER:
        np.testing.assert_array_equal(_bits(np.asarray(got[key])), _bits(want[key]), err_msg=key)
    for key, atol in CLOSE_RASTER.items():
        np.testing.assert_allclose(got[key], want[key], rtol=RTOL, atol=atol, err_msg=key)


EXACT_GAUSSIAN = EXACT_RASTER + ("conic", "image", "alpha")   # one fixed fp32 sequence for the footprint on both sides
CLOSE_GAUSSIAN = {"blending_weights": 1e-7, "grad_features": 2e-7, "grad_opacities": 1e-6}


def test_oracle_reproduces_gaussian_fixture(oracle, maker):
    want = np.load(GOLDEN / "gaussian_small.npz")
    got = maker.gaussian_answers()
    for key in EXACT_GAUSSIAN:
        np.testing.assert_array_equal(_bits(np.asarray(got[key])), _bits(want[key]), err_msg=key)
    for key, atol in CLOSE_GAUSSIAN.items():
        np.testing.assert_allclose(got[key], want[key], rtol=RTOL, atol=atol, err_msg=key)


@pytest.mark.gpu
def test_hip_gaussian_footprint_gives_fixture(gpu, maker):
    from inpc_amd import _lib
    from tests import helpers as H

    want = np.load(GOLDEN / "gaussian_small.npz")
    p = maker.RASTER
    hv, pos, feats, opac, gi, ga = maker.raster_case()
    run = H.GaussianRun(hv, pos, feats, opac, 8, p["channels"], _lib.FEAT_DIRECT_F32).forward()
    dbg = run.debug()
    out = run.outputs()
    for key in EXACT_GAUSSIAN:
        got = np.asarray(out[key] if key in out else dbg[key])
        np.testing.assert_array_equal(_bits(got), _bits(want[key]), err_msg=key)
    H.assert_close(out["blending_weights"], want["blending_weights"], RTOL, CLOSE_GAUSSIAN["blending_weights"], "weights")
    gf, go = run.backward(gi, ga)
    H.assert_close(gf, want["grad_features"], RTOL, CLOSE_GAUSSIAN["grad_features"], "feature gradients")
    H.assert_close(go, want["grad_opacities"], RTOL, CLOSE_GAUSSIAN["grad_opacities"], "opacity gradients")


@pytest.mark.gpu
def test_hip_sampler_gives_fixture(gpu, maker):
    import torch

    from inpc_amd import ProbabilityFieldSampler
    from tests import helpers as H

    want = np.load(GOLDEN / "sampler_small.npz")
    p = maker.SAMPLER
    oct, hv = maker.sampler_case()
    w = H.leaf_weights(oct, hv)
    np.testing.assert_array_equal(_bits(w.cpu().numpy()), _bits(want["leaf_weights"]))
    cdf, head = H.build_cdf(w)
    np.testing.assert_array_equal(_bits(cdf.cpu().numpy()), _bits(want["cdf"]))
    assert _bits(head[:1].cpu().numpy())[0] == _bits(want["total"].reshape(1))[0]
    rng = H.make_rng(p["rng_seed"])
    pos, ids = H.sample(oct, cdf, head, p["n_plain"], rng)
    np.testing.assert_array_equal(ids, want["plain_ids"])
    np.testing.assert_array_equal(_bits(pos), _bits(want["plain_positions"]))
    assert H.rng_values(rng) == tuple(int(v) for v in want["plain_state"])
    # the whole training draw through the operator layer
    sampler = ProbabilityFieldSampler(seed=p["rng_seed"])
    view = hv.to_view(gpu)
    tpos, tids = sampler.generate_training_samples(H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights), view,
                                                   p["n_training"], oct.initial_size)
    np.testing.assert_array_equal(tids.cpu().numpy(), want["training_ids"].astype(np.int64))
    np.testing.assert_array_equal(_bits(tpos.cpu().numpy()), _bits(want["training_positions"]))


@pytest.mark.gpu
def test_hip_rasterizer_gives_fixture(gpu, maker):
    from inpc_amd import _lib
    from tests import helpers as H

    want = np.load(GOLDEN / "raster_small.npz")
    p = maker.RASTER
    hv, pos, feats, opac, gi, ga = maker.raster_case()
    run = H.RasterRun(hv, pos, feats, opac, p["tile"], p["channels"], _lib.FEAT_DIRECT_F32).forward()
    dbg = run.debug()
    for key in EXACT_RASTER:
        if key in ("depth_keys", "depth_order"):
            continue   # the fixture's device-wide depth order; here every tile's instances are sorted on their own
        got = np.asarray(dbg[key])
        if key in ("instance_keys", "instance_points"):
            got = got[: len(want[key])]
        np.testing.assert_array_equal(_bits(got), _bits(want[key]), err_msg=key)
    key_of_point = np.zeros(len(want["n_touched"]), np.uint32)
    key_of_point[want["depth_order"]] = want["depth_keys"]
    np.testing.assert_array_equal(dbg["instance_depth_keys"], key_of_point[want["instance_points"]])
    out = run.outputs()
    for key in ("image", "alpha", "blending_weights"):
        H.assert_close(out[key], want[key], RTOL, CLOSE_RASTER[key], key)
    gf, go = run.backward(gi, ga)
    H.assert_close(gf, want["grad_features"], RTOL, CLOSE_RASTER["grad_features"], "feature gradients")
    H.assert_close(go, want["grad_opacities"], RTOL, CLOSE_RASTER["grad_opacities"], "opacity gradients")
