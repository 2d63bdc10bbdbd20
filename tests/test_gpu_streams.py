"""Calls in flight on several streams at once, with a workspace each: the kernels that wait for each other's tiles
(the sampler's cull kernels) hand their tiles out through tickets, so they do not depend on owning the GPU; the
rasterizer has no such kernel. Every result is compared with the oracle and every device error flag must be clear."""
import numpy as np
import pytest
import torch

from inpc_amd import _lib, synthetic
from tests import helpers as H
from tests.test_gpu_gaussian import check_structure as check_gaussian_structure, grad_atol, oracle_run
from tests.test_gpu_raster import check_structure, oracle_cfg

pytestmark = [pytest.mark.gpu, pytest.mark.real_gpu]

RTOL = 1e-4


def test_forward_backward_on_three_streams_at_once(gpu, oracle):
    n, channels = 400000, 8
    cases = []
    for k in range(3):
        hv = synthetic.rotated_camera(400 + 16 * k, 300, 330.0, 2.6, 0.1 * k, -0.05 * k)
        pos = synthetic.cube_points(n, 1.8, 40 + k)
        feats, opac = synthetic.point_attributes(n, channels, "normal", 50 + k)
        rng = np.random.default_rng(60 + k)
        gi = rng.normal(0, 1e-2, (channels, hv.camera.height, hv.camera.width)).astype(np.float32)
        ga = rng.normal(0, 1e-2, (1, hv.camera.height, hv.camera.width)).astype(np.float32)
        cases.append((hv, pos, feats, opac, gi, ga))
    streams = [torch.cuda.Stream() for _ in cases]
    runs, grads = [], []
    torch.cuda.synchronize()
    # enqueue everything first, read back afterwards: the three calls overlap on the device
    for k, (stream, (hv, pos, feats, opac, gi, ga)) in enumerate(zip(streams, cases)):
        with torch.cuda.stream(stream):
            if k == 2:   # one call with the bilinear footprint among the two Gaussian ones
                run = H.RasterRun(hv, pos, feats, opac, 16, channels, _lib.FEAT_DIRECT_F32)
            else:
                run = H.GaussianRun(hv, pos, feats, opac, 8, channels, _lib.FEAT_DIRECT_F32)
            runs.append(run)
    for stream, run in zip(streams, runs):
        with torch.cuda.stream(stream):
            run.forward()
    for stream, run, case in zip(streams, runs, cases):
        with torch.cuda.stream(stream):
            gi_dev, ga_dev = H.dev(case[4]), H.dev(case[5])
            grads.append(run.backward_async(gi_dev, ga_dev))
    torch.cuda.synchronize()
    for k, (run, (hv, pos, feats, opac, gi, ga), (gf, go)) in enumerate(zip(runs, cases, grads)):
        out = run.outputs()
        if k == 2:
            cfg = oracle_cfg(oracle, hv, n, 16, channels, oracle.FEAT_DIRECT_F32)
            ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
            check_structure(run.debug(), ref)       # reads the counters: the device error flag is clear
            gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
        else:
            g, ref = oracle_run(oracle, hv, pos, feats, opac, 8, channels)
            check_gaussian_structure(run.debug(), ref)
            gf_ref, go_ref, _ = oracle.raster_backward(g.base, gi, ga, out["image"], out["alpha"], pos, feats, opac,
                                                       hv.w2c, gaussian=g)
        H.assert_close(out["image"], ref["image"], RTOL, 1e-5, f"image {k}")
        H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, f"blending weights {k}")
        H.assert_close(gf.cpu().numpy(), gf_ref, RTOL, grad_atol(gf_ref), f"feature gradients {k}")
        H.assert_close(go.cpu().numpy(), go_ref, RTOL, grad_atol(go_ref), f"opacity gradients {k}")


def test_training_draws_on_two_streams_at_once(gpu, oracle):
    from inpc_amd import ProbabilityFieldSampler

    oct = synthetic.octree_leaves(40000, 7, 4.0, seed=3)
    views = [synthetic.camera_on_z(320, 200, 260.0, 6.0), synthetic.rotated_camera(300, 220, 250.0, 6.0, 0.3, 0.1)]
    n = 600000
    streams = [torch.cuda.Stream() for _ in views]
    samplers = [ProbabilityFieldSampler(seed=11 + k) for k in range(2)]
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    torch.cuda.synchronize()
    # a draw reads its counts back, so each runs on a host thread of its own to be in flight together with the other
    import threading

    results = [None, None]

    def draw(k):
        with torch.cuda.stream(streams[k]):
            results[k] = samplers[k].generate_training_samples(centers, levels, weights, views[k].to_view(gpu), n,
                                                               oct.initial_size)

    threads = [threading.Thread(target=draw, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for k, ((pos, ids), hv) in enumerate(zip(results, views)):
        c = hv.camera
        cam = oracle.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)
        pos_ref, ids_ref, _ = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c, cam,
                                                      oct.initial_size, oracle.Pcg32(11 + k), n)
        np.testing.assert_array_equal(ids.cpu().numpy(), ids_ref.astype(np.int64))
        np.testing.assert_array_equal(pos.cpu().numpy().view(np.uint32), pos_ref.view(np.uint32))


def test_bilinear_steps_from_four_host_threads_share_the_second_stream(gpu, oracle):
    """The bilinear forward pass writes its records on a second stream that all calls on the device share: four
    host threads, a stream and a workspace each, several steps each, all in flight together."""
    import threading

    n, channels, steps = 150000, 8, 4
    cases = []
    for k in range(4):
        hv = synthetic.rotated_camera(320 + 16 * k, 240, 300.0, 2.6, 0.07 * k, -0.04 * k)
        pos = synthetic.cube_points(n, 1.8, 70 + k)
        feats, opac = synthetic.point_attributes(n, channels, "normal", 80 + k)
        rng = np.random.default_rng(90 + k)
        gi = rng.normal(0, 1e-2, (channels, hv.camera.height, hv.camera.width)).astype(np.float32)
        ga = rng.normal(0, 1e-2, (1, hv.camera.height, hv.camera.width)).astype(np.float32)
        cases.append((hv, pos, feats, opac, gi, ga))
    H.RasterRun(*cases[0][:4], 16, channels, _lib.FEAT_DIRECT_F32).forward()   # the second stream exists from here on
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in cases]
    results = [None] * len(cases)
    errors = []

    def work(k):
        try:
            hv, pos, feats, opac, gi, ga = cases[k]
            with torch.cuda.stream(streams[k]):
                run = H.RasterRun(hv, pos, feats, opac, 16 if k % 2 == 0 else 8, channels, _lib.FEAT_DIRECT_F32)
                gi_dev, ga_dev = H.dev(gi), H.dev(ga)
                for _ in range(steps):
                    run.forward()
                    grads = run.backward_async(gi_dev, ga_dev)
                streams[k].synchronize()
            results[k] = (run, grads)
        except Exception as exc:   # reported by the main thread
            errors.append((k, exc))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for k, ((run, (gf, go)), (hv, pos, feats, opac, gi, ga)) in enumerate(zip(results, cases)):
        tile = 16 if k % 2 == 0 else 8
        cfg = oracle_cfg(oracle, hv, n, tile, channels, oracle.FEAT_DIRECT_F32)
        ref = oracle.raster_forward(cfg, pos, feats, opac, hv.w2c, debug=True)
        check_structure(run.debug(), ref)
        out = run.outputs()
        H.assert_close(out["image"], ref["image"], RTOL, 1e-5, f"image {k}")
        H.assert_close(out["blending_weights"], ref["blending_weights"], RTOL, 1e-7, f"blending weights {k}")
        gf_ref, go_ref, _ = oracle.raster_backward(cfg, gi, ga, out["image"], out["alpha"], pos, feats, opac, hv.w2c)
        H.assert_close(gf.cpu().numpy(), gf_ref, RTOL, grad_atol(gf_ref), f"feature gradients {k}")
        H.assert_close(go.cpu().numpy(), go_ref, RTOL, grad_atol(go_ref), f"opacity gradients {k}")
