"""Writes the golden fixtures of this directory from the CPU oracle.

The reference ships no vectors for the sampling / rasterization path and cannot run here (CUDA sources), so these
fixtures do not come from it: they freeze the oracle's answers on three small seeded cases, so that a later change of
the oracle (or of the canonical rules it encodes) shows up as a diff of committed data, and so that the HIP path is
checked against data as well as against the oracle built from today's sources.

    python tests/golden/make_golden.py          # rewrites sampler_small.npz, raster_small.npz, gaussian_small.npz
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from inpc_amd import synthetic  # noqa: E402  (host-side scene generators, no GPU)
from oracle import oracle as O  # noqa: E402

HERE = Path(__file__).resolve().parent

SAMPLER = dict(n_leaves=2048, level=5, extent=4.0, seed=3, width=160, height=120, focal=140.0, distance=6.0,
               rng_seed=17, n_plain=3000, n_training=2500)
RASTER = dict(n=6000, channels=4, tile=16, width=96, height=64, focal=90.0, distance=2.4, side=1.6, seed=5)


def sampler_case():
    p = SAMPLER
    oct = synthetic.octree_leaves(p["n_leaves"], p["level"], p["extent"], seed=p["seed"])
    hv = synthetic.camera_on_z(p["width"], p["height"], p["focal"], p["distance"])
    return oct, hv


def raster_case():
    p = RASTER
    hv = synthetic.camera_on_z(p["width"], p["height"], p["focal"], p["distance"])
    pos = synthetic.cube_points(p["n"], p["side"], p["seed"])
    feats, opac = synthetic.point_attributes(p["n"], p["channels"], "normal", p["seed"] + 1, np.float32)
    rng = np.random.default_rng(p["seed"] + 2)
    gi = rng.normal(0, 1e-2, (p["channels"], p["height"], p["width"])).astype(np.float32)
    ga = rng.normal(0, 1e-2, (1, p["height"], p["width"])).astype(np.float32)
    return hv, pos, feats, opac, gi, ga


def oracle_camera(hv):
    c = hv.camera
    return O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)


def sampler_answers():
    p = SAMPLER
    oct, hv = sampler_case()
    cam = oracle_camera(hv)
    w = O.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam, oct.initial_size)
    ok, cdf, total = O.build_cdf(w)
    assert ok
    rng = O.Pcg32(p["rng_seed"])
    pos_plain, ids_plain = O.sample(oct.centers, oct.levels, cdf, p["n_plain"], oct.initial_size, rng)
    state_plain = np.array(rng.state, np.uint64)
    rng = O.Pcg32(p["rng_seed"])
    pos_train, ids_train, consumed = O.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c, cam,
                                                        oct.initial_size, rng, p["n_training"])
    return dict(leaf_weights=w, cdf=cdf, total=np.float32(total), plain_positions=pos_plain, plain_ids=ids_plain,
                plain_state=state_plain, training_positions=pos_train, training_ids=ids_train,
                training_consumed=np.int64(consumed), training_state=np.array(rng.state, np.uint64))


def raster_answers():
    p = RASTER
    hv, pos, feats, opac, gi, ga = raster_case()
    cfg = O.make_config(p["n"], oracle_camera(hv), p["tile"], p["channels"], O.FEAT_DIRECT_F32, 0)
    ref = O.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
    gf, go, _ = O.raster_backward(cfg, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c)
    keep = ("n_visible", "n_instances", "n_touched", "bounds", "screen_xy", "depth_keys", "depth_order",
            "instance_keys", "instance_points", "tile_ranges", "image", "alpha", "blending_weights")
    out = {k: np.asarray(ref[k]) for k in keep}
    out.update(grad_features=gf, grad_opacities=go)
    return out


def gaussian_answers():
    """The raster case through the Gaussian footprint (training variance), 8x8 tiles."""
    p = RASTER
    hv, pos, feats, opac, gi, ga = raster_case()
    base = O.make_config(p["n"], oracle_camera(hv), 8, p["channels"], O.FEAT_DIRECT_F32, 0)
    g = O.GaussianConfig(base, 0.0, 3.0, 0, 0)
    count = O.gaussian_instance_count(g, pos, hv.w2c)
    ref = O.raster_forward(base, pos, feats, opac, hv.w2c, debug=True, gaussian=g, n_instances_hint=count)
    gf, go, _ = O.raster_backward(base, gi, ga, ref["image"], ref["alpha"], pos, feats, opac, hv.w2c, gaussian=g)
    keep = ("n_visible", "n_instances", "n_touched", "bounds", "screen_xy", "conic", "depth_keys", "depth_order",
            "instance_keys", "instance_points", "tile_ranges", "image", "alpha", "blending_weights")
    out = {k: np.asarray(ref[k]) for k in keep}
    out.update(grad_features=gf, grad_opacities=go)
    return out


def main():
    np.savez_compressed(HERE / "sampler_small.npz", **sampler_answers())
    np.savez_compressed(HERE / "raster_small.npz", **raster_answers())
    np.savez_compressed(HERE / "gaussian_small.npz", **gaussian_answers())
    for name in ("sampler_small.npz", "raster_small.npz", "gaussian_small.npz"):
        print(name, (HERE / name).stat().st_size, "bytes")


if __name__ == "__main__":
    main()
