#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

One step = one rasterizer forward + backward over 8,388,608 points at 1237x822 (8 fp32 channels,
16x16 tiles), the configuration the headline metric is quoted on. The points are drawn on the GPU by the
sampler (262,144 log-normal leaves of a depth-9 octree over [-2,2]^3, camera at (0,0,-6), f = 1000);
features ~N(0,1), opacity = sigmoid(N(0,1)), image gradients ~N(0,1e-2). All inputs are resident in HBM
before the timed region.

Prints ONE JSON line. `value` is Mpoints/s of forward+backward; `roofline` describes the kernel with the
largest share of the step (algorithmic bytes per launch / HIP-event duration on the launch stream);
`cpu_baseline` is the CPU oracle running the same step on a bounded sample, with all host threads and with one.
`extra` carries the sampler's figures, the Gaussian footprint, the reference-shaped autograd step, BASELINE
configuration 0, the reference's default inference frame and the large-frame inference configuration (33,554,432
points @2473x1643). `--only-config4` runs that last configuration alone and prints it as the one line, so that a
profiler run of it holds no kernel of the training step.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    # name: (n_points, width, height, focal, channels, tile, n_leaves, level)
    "config3": dict(n=8_388_608, width=1237, height=822, focal=1000.0, channels=8, tile=16, leaves=262_144, level=9,
                    describe="rasterizer fwd+bwd, 8,388,608 pts @1237x822, C=8 fp32, 16x16 tiles"),
    "config3_t8": dict(n=8_388_608, width=1237, height=822, focal=1000.0, channels=8, tile=8, leaves=262_144, level=9,
                       describe="rasterizer fwd+bwd, 8,388,608 pts @1237x822, C=8 fp32, 8x8 tiles"),
    "small": dict(n=262_144, width=640, height=400, focal=500.0, channels=8, tile=16, leaves=32_768, level=7,
                  describe="rasterizer fwd+bwd, 262,144 pts @640x400, C=8 fp32, 16x16 tiles (quick check)"),
}

# Sizes of the side measurements of `extra` (module-level so that tests/test_bench_dry_run.py can shrink them).
DEVICE = "cuda:0"
CONFIG0_POINTS = 65_536                     # BASELINE configuration 0: the reference's CPU-sized case
FRAME_REQUESTED_SAMPLES = 8_388_352         # per sampling round of the reference's default inference frame
CONFIG4 = dict(n=33_554_432, width=2473, height=1643, focal=2000.0, leaves=2_097_152, level=11)


def algorithmic_bytes(kernel: str, n, v, i, pixels, channels, end_bit):
    """Algorithmic bytes that all launches of `kernel` in one step move together: every array of the reference's
    pipeline structure touched the minimum number of times that structure requires, booked on the kernel that does
    that part of the work here. F = feature bytes per point, R = blend record (8 xy + 4 opacity + 4C features).
    Kernels that only exist in this pipeline (bin offsets, the gradient reduction) carry no algorithmic bytes."""
    F = 4 * channels
    R = 8 + 4 + 4 * channels
    table = {
        # the count/scan in front of the instance expansion
        "raster_bin_count": v * 20,
        # point in (xyz, features, opacity), record out
        "raster_records": n * (16 + F) + v * R,
        # key/index out, instance emission (expansion reads + 6 B each)
        "raster_bin_fill": v * (8 + 16) + i * 6,
        # what the reference structure spends on ordering: depth sort of the visible points (4 B histogram read +
        # 4 passes x 16 B), tile sort of the instances and the range scan
        "raster_tile_sort": v * 68 + i * (2 + 12 * ((end_bit + 7) // 8) + 2),
        "raster_blend_forward": i * (4 + R) + pixels * 4 * (channels + 1) + n * 4,
        "raster_blend_backward": i * (4 + R) + pixels * 8 * (channels + 1) + n * (4 * channels + 4),
        "fill_u32": n * (4 * channels + 4),
    }
    return float(table.get(kernel, 0.0))


def traffic_file(workload: str) -> Path:
    return ROOT / "profiles" / f"hbm_traffic_{workload}.txt"


def measured_traffic(kernel: str, workload: str):
    """HBM bytes per launch of `kernel` from the committed profiler-counter summary of this workload
    (profiles/hbm_traffic_<workload>.txt, lines `<kernel> fetch_bytes=F write_bytes=W total_bytes=T`),
    or None when no such measurement is on file. The figure comes from that earlier profiler run of the same
    command, not from the run that prints it."""
    path = traffic_file(workload)
    if not path.exists():
        return None
    for line in path.read_text().splitlines():
        parts = line.split()
        if parts and parts[0] == kernel:
            for item in parts[1:]:
                if item.startswith("total_bytes="):
                    return float(item.split("=", 1)[1])
    return None


def step_algorithmic_bytes(n, v, i, pixels, channels, end_bit):
    """Whole forward + backward step under the same model."""
    R = 8 + 4 + 4 * channels
    fwd = n * (16 + 4 * channels) + v * (R + 8 + 68 + 20 + 16) + n * 4 \
        + i * (6 + 2 + 12 * ((end_bit + 7) // 8) + 2 + 4 + R) + pixels * 4 * (channels + 1)
    bwd = i * (4 + R) + pixels * 8 * (channels + 1) + n * 2 * (4 * channels + 4)
    return float(fwd), float(bwd)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="config3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also launch three 1 GiB plain copies (the yardstick for profiler byte counters)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target duration of the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="only the timed step, its per-kernel durations and the sampler draw: no graph replay, field "
                         "update, Gaussian footprint, reference-shaped step or large-frame leg (for profiler runs)")
    ap.add_argument("--no-config4", action="store_true",
                    help="skip the large-frame inference configuration (33,554,432 points @2473x1643, 16 fp16 "
                         "channels: training draw + inference forward, reported in extra.config4_inference)")
    ap.add_argument("--only-config4", action="store_true",
                    help="only the large-frame inference configuration, as the one JSON line (for profiler runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; --gpus N with N > 1 is not supported "
              "(the path runs on a single GPU)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from inpc_amd import ProbabilityFieldSampler, _lib, synthetic

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    lib = _lib.lib()
    device = torch.device(DEVICE)
    torch.cuda.set_device(device)
    wl = WORKLOADS[args.workload]
    n, channels, tile = wl["n"], wl["channels"], wl["tile"]
    stream = _lib.current_stream()
    gen = torch.Generator(device=device).manual_seed(1)

    def time_calls(fn, reps):
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e3 / reps

    def config4_leg():
        """BASELINE configuration 4: the large frame's training draw and its inference forward pass (both footprints
        through the operator layer, the bilinear one once more through the C ABI with per-kernel figures)."""
        n4, W4, H4 = CONFIG4["n"], CONFIG4["width"], CONFIG4["height"]
        hv4 = synthetic.camera_on_z(W4, H4, CONFIG4["focal"], 6.0)
        view4 = hv4.to_view(device)
        oct4 = synthetic.octree_leaves(CONFIG4["leaves"], CONFIG4["level"], 4.0, seed=0)
        c4, l4, w4 = (torch.from_numpy(a).to(device) for a in (oct4.centers, oct4.levels, oct4.weights))
        sampler4 = ProbabilityFieldSampler(seed=0)
        pos4, _ = sampler4.generate_training_samples(c4, l4, w4, view4, n4, oct4.initial_size)
        draw4_ms = time_calls(lambda: sampler4.generate_training_samples(c4, l4, w4, view4, n4, oct4.initial_size), 5)
        feats4 = torch.randn((n4, 16), generator=gen, device=device, dtype=torch.float32).half()
        opac4 = torch.sigmoid(torch.randn(n4, generator=gen, device=device, dtype=torch.float32))
        config4 = {"workload": f"{n4:,} pts @{W4}x{H4}, 16 channels stored fp16, inference forward",
                   "training_draw_ms": round(draw4_ms, 3)}
        from inpc_amd import rasterize_points

        for label, mode, tile4, kw in (("bilinear", 0, 16, {}),
                                       ("gaussian", 1, 8, dict(sigma_world=0.002, sigma_cutoff=3.0))):
            def infer():
                rasterize_points(view4, pos4, feats4, opac4, tile=tile4, inference=True, mode=mode, **kw)

            infer()
            ms = time_calls(infer, 5)
            config4[f"{label}_forward_ms"] = round(ms, 3)
            config4[f"{label}_Mpoints_per_s"] = round(n4 / (ms * 1e-3) / 1e6, 1)
        # the bilinear forward once more through the C ABI: its counts, per-kernel durations (HIP events on the launch
        # stream) and the share of the HBM roofline of the frame and of its largest kernel. Algorithmic bytes as for
        # the training step, with 2 bytes per stored feature.
        try:
            cfg4 = _lib.RasterConfig(n4, 16, 16, _lib.FEAT_DIRECT_F16, _lib.RASTER_INFERENCE, _lib.make_camera(hv4.camera), 0)
            layout4 = _lib.RasterLayout()
            _lib.check(lib.inpc_raster_layout_query(C.byref(cfg4), C.byref(layout4)), "layout")
            ws4 = torch.empty(layout4.total_bytes, dtype=torch.uint8, device=device)
            image4 = torch.empty((16, H4, W4), dtype=torch.float32, device=device)
            alpha4 = torch.empty((1, H4, W4), dtype=torch.float32, device=device)
            depth4 = torch.empty((1, H4, W4), dtype=torch.float32, device=device)
            w2c4, camp4 = view4.w2c.contiguous(), view4.position.contiguous()

            def forward4():
                _lib.check(lib.inpc_raster_forward(C.byref(cfg4), _lib.ptr(pos4), _lib.ptr(feats4), _lib.ptr(opac4),
                                                   _lib.ptr(w2c4), _lib.ptr(camp4), _lib.ptr(image4), _lib.ptr(alpha4), None,
                                                   _lib.ptr(depth4), _lib.ptr(ws4), layout4.total_bytes, stream),
                           "inpc_raster_forward")

            forward4()
            counters4 = (C.c_uint32 * 3)()
            _lib.check(lib.inpc_raster_read_counters(C.byref(cfg4), _lib.ptr(ws4), C.byref(counters4), stream), "counters")
            v4, i4 = int(counters4[0]), int(counters4[1])
            abi_ms = time_calls(forward4, 5)
            with _lib.KernelTimer() as timer4:
                for _ in range(3):
                    forward4()
            k4 = {}
            for name, ms in timer4.records:
                tot, cnt = k4.get(name, (0.0, 0))
                k4[name] = (tot + ms, cnt + 1)
            F4, R4, px4 = 2 * 16, 8 + 4 + 2 * 16, H4 * W4
            sort_bytes = 2 + 12 * ((layout4.end_bit + 7) // 8) + 2
            frame_bytes = float(n4 * (16 + F4) + v4 * (R4 + 8 + 68 + 20 + 16) + i4 * (6 + sort_bytes + 4 + R4)
                                + px4 * 4 * (16 + 2))
            per_kernel_bytes = {
                "raster_bin_count": v4 * 20.0, "raster_records": float(n4 * (16 + F4) + v4 * R4),
                "raster_bin_fill": float(v4 * (8 + 16) + i4 * 6), "raster_tile_sort": float(v4 * 68 + i4 * sort_bytes),
                "raster_blend_inference": float(i4 * (4 + R4) + px4 * 4 * (16 + 2)),
            }
            rows4 = []
            for name, (tot, cnt) in sorted(k4.items(), key=lambda kv: -kv[1][0]):
                launches = cnt / 3
                avg = tot / cnt
                alg = per_kernel_bytes.get(name, 0.0) / launches
                rows4.append({"kernel": name, "launches_per_frame": launches, "avg_ms": round(avg, 4),
                              "ms_per_frame": round(tot / 3, 4),
                              "algorithmic_GBps": round(alg / (avg * 1e-3) / 1e9, 1) if alg > 0 and avg > 0 else None})
            top = rows4[0]
            top_alg = per_kernel_bytes.get(top["kernel"], 0.0) / top["launches_per_frame"]
            top_gbps = top_alg / (top["avg_ms"] * 1e-3) / 1e9
            config4["bilinear_abi"] = {
                "forward_ms": round(abi_ms, 3), "n_visible": v4, "n_instances": i4, "n_tiles": int(layout4.n_tiles),
                "frame_algorithmic_GB": round(frame_bytes / 1e9, 3),
                "frame_hbm_frac": round(frame_bytes / (abi_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "roofline": {"bound": "hbm", "kernel": top["kernel"], "achieved": round(top_gbps, 1),
                             "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(top_gbps / HBM_PEAK_GBS, 4),
                             "algorithmic_bytes_per_launch": top_alg, "avg_launch_ms": top["avg_ms"],
                             "traffic": measured_traffic(top["kernel"], "config4")},
                "kernels": rows4}
            del ws4, image4, alpha4, depth4
        except Exception as exc:  # the figure is optional
            print(f"bench.py: config-4 per-kernel figures not measured: {exc}", file=sys.stderr)

        return config4

    if args.only_config4:
        # the large frame alone (for profiler runs that must not mix its kernels with the training step's)
        config4 = config4_leg()
        abi = config4.get("bilinear_abi") or {}
        ms = abi.get("forward_ms", config4["bilinear_forward_ms"])
        print(json.dumps({
            "metric": "Mpoints/s, inference forward of the large frame (ms/frame in ms_per_step)",
            "value": round(CONFIG4["n"] / (ms * 1e-3) / 1e6, 1), "unit": "Mpoints/s", "n_gpus": 1, "steps": 5, "warmup": 1,
            "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic", "config": {"workload": config4["workload"]}, "roofline": abi.get("roofline"),
            "cpu_baseline": None, "extra": {"config4_inference": config4}}))
        return 0


    # ---- inputs ---------------------------------------------------------------------------------------
    hv = synthetic.camera_on_z(wl["width"], wl["height"], wl["focal"], 6.0)
    view = hv.to_view(device)
    oct = synthetic.octree_leaves(wl["leaves"], wl["level"], 4.0, seed=0)
    centers = torch.from_numpy(oct.centers).to(device)
    levels = torch.from_numpy(oct.levels).to(device)
    weights = torch.from_numpy(oct.weights).to(device)
    sampler = ProbabilityFieldSampler(seed=0)
    draws = []   # a training draw as the loop sees it: wall time of the call, the sampler's estimates settled
    for _ in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
        torch.cuda.synchronize()
        draws.append((time.perf_counter() - t0) * 1e3)
    sampler_ms = sorted(draws[1:])[len(draws[1:]) // 2]
    with _lib.KernelTimer() as draw_timer:   # the kernels of one more draw, HIP events on the launch stream
        sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
    draw_kernels = {}
    for name, ms in draw_timer.records:
        draw_kernels[name] = draw_kernels.get(name, 0.0) + ms
    draw_candidates = int(sampler.last_consumed)
    sampler = ProbabilityFieldSampler(seed=0)   # the benchmark's points: the first draw of seed 0
    positions, leaf_ids = sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
    torch.cuda.synchronize()

    features = torch.randn((n, channels), generator=gen, device=device, dtype=torch.float32)
    opacities = torch.sigmoid(torch.randn(n, generator=gen, device=device, dtype=torch.float32))
    H, W = wl["height"], wl["width"]
    grad_image = torch.randn((channels, H, W), generator=gen, device=device) * 1e-2
    grad_alpha = torch.randn((1, H, W), generator=gen, device=device) * 1e-2

    cfg = _lib.RasterConfig(n, tile, channels, _lib.FEAT_DIRECT_F32, 0, _lib.make_camera(hv.camera))
    layout = _lib.RasterLayout()
    _lib.check(lib.inpc_raster_layout_query(C.byref(cfg), C.byref(layout)), "layout")
    workspace = torch.empty(layout.total_bytes, dtype=torch.uint8, device=device)
    image = torch.empty((channels, H, W), dtype=torch.float32, device=device)
    alpha = torch.empty((1, H, W), dtype=torch.float32, device=device)
    blending_weights = torch.empty(n, dtype=torch.float32, device=device)
    grad_features = torch.empty((n, channels), dtype=torch.float32, device=device)
    grad_opacities = torch.empty(n, dtype=torch.float32, device=device)
    w2c, cam_position = view.w2c.contiguous(), view.position.contiguous()

    def forward():
        _lib.check(lib.inpc_raster_forward(C.byref(cfg), _lib.ptr(positions), _lib.ptr(features), _lib.ptr(opacities),
                                           _lib.ptr(w2c), _lib.ptr(cam_position), _lib.ptr(image), _lib.ptr(alpha),
                                           _lib.ptr(blending_weights), None, _lib.ptr(workspace), layout.total_bytes,
                                           stream), "inpc_raster_forward")

    def backward():
        _lib.check(lib.inpc_raster_backward(C.byref(cfg), _lib.ptr(grad_image), _lib.ptr(grad_alpha), _lib.ptr(image),
                                            _lib.ptr(alpha), _lib.ptr(positions), _lib.ptr(cam_position),
                                            _lib.ptr(grad_features), _lib.ptr(grad_opacities), None,
                                            _lib.ptr(workspace), layout.total_bytes, stream), "inpc_raster_backward")

    def step():
        forward()
        backward()

    if args.pmc_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(lib.inpc_calibration_copy(_lib.ptr(src), _lib.ptr(dst), src.numel(), stream), "copy")
        torch.cuda.synchronize()
        del src, dst

    # ---- timed region ---------------------------------------------------------------------------------
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    counters = (C.c_uint32 * 3)()
    _lib.check(lib.inpc_raster_read_counters(C.byref(cfg), _lib.ptr(workspace), C.byref(counters), stream), "counters")
    n_visible, n_instances = int(counters[0]), int(counters[1])

    # forward alone / backward alone
    fwd_ms = time_calls(forward, args.steps)
    bwd_ms = time_calls(backward, args.steps)

    # the same step replayed from a graph (the library only enqueues kernels, so a caller may capture it):
    # what is left of the step when the host's launch work is taken away
    graph_ms = None
    try:
        if args.no_extras:
            raise RuntimeError("skipped (--no-extras)")
        side = torch.cuda.Stream()

        def step_on_current_stream():
            s = _lib.current_stream()
            _lib.check(lib.inpc_raster_forward(C.byref(cfg), _lib.ptr(positions), _lib.ptr(features), _lib.ptr(opacities),
                                               _lib.ptr(w2c), _lib.ptr(cam_position), _lib.ptr(image), _lib.ptr(alpha),
                                               _lib.ptr(blending_weights), None, _lib.ptr(workspace), layout.total_bytes,
                                               s), "inpc_raster_forward")
            _lib.check(lib.inpc_raster_backward(C.byref(cfg), _lib.ptr(grad_image), _lib.ptr(grad_alpha), _lib.ptr(image),
                                                _lib.ptr(alpha), _lib.ptr(positions), _lib.ptr(cam_position),
                                                _lib.ptr(grad_features), _lib.ptr(grad_opacities), None,
                                                _lib.ptr(workspace), layout.total_bytes, s), "inpc_raster_backward")

        # one eager step on the stream first: the library gives a stream its second stream (for the blend records)
        # the first time it sees the stream outside a capture
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            step_on_current_stream()
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step_on_current_stream()
        graph.replay()
        graph_ms = time_calls(graph.replay, args.steps)
    except Exception as exc:  # the figure is optional
        print(f"bench.py: graph replay not measured: {exc}", file=sys.stderr)

    # the step that closes the loop: leaf statistics from this frame's leaf indices and blending weights
    from inpc_amd import update_probability_field

    field_ms = None
    if not args.no_extras:
        field_weights = weights.clone()
        field_scores = torch.zeros_like(weights)
        field_ms = time_calls(lambda: update_probability_field(field_weights, field_scores, leaf_ids, blending_weights),
                              args.steps)

    # the same step with the other tile size (the reference's tiles are 8x8; the images do not depend on the tile size):
    # a side measurement, not part of `value`
    other_tile = None
    if not args.no_extras:
        t2 = 8 if tile == 16 else 16
        cfg2 = _lib.RasterConfig(n, t2, channels, _lib.FEAT_DIRECT_F32, 0, _lib.make_camera(hv.camera), 0)
        layout2 = _lib.RasterLayout()
        _lib.check(lib.inpc_raster_layout_query(C.byref(cfg2), C.byref(layout2)), "layout")
        ws2 = torch.empty(layout2.total_bytes, dtype=torch.uint8, device=device)
        image2, alpha2, bw2 = torch.empty_like(image), torch.empty_like(alpha), torch.empty_like(blending_weights)
        gf2, go2 = torch.empty_like(grad_features), torch.empty_like(grad_opacities)

        def step2():
            _lib.check(lib.inpc_raster_forward(C.byref(cfg2), _lib.ptr(positions), _lib.ptr(features), _lib.ptr(opacities),
                                               _lib.ptr(w2c), _lib.ptr(cam_position), _lib.ptr(image2), _lib.ptr(alpha2),
                                               _lib.ptr(bw2), None, _lib.ptr(ws2), layout2.total_bytes, stream),
                       "inpc_raster_forward")
            _lib.check(lib.inpc_raster_backward(C.byref(cfg2), _lib.ptr(grad_image), _lib.ptr(grad_alpha), _lib.ptr(image2),
                                                _lib.ptr(alpha2), _lib.ptr(positions), _lib.ptr(cam_position), _lib.ptr(gf2),
                                                _lib.ptr(go2), None, _lib.ptr(ws2), layout2.total_bytes, stream),
                       "inpc_raster_backward")

        step2()
        step2_ms = time_calls(step2, args.steps)
        counters2 = (C.c_uint32 * 3)()
        _lib.check(lib.inpc_raster_read_counters(C.byref(cfg2), _lib.ptr(ws2), C.byref(counters2), stream), "counters")
        other_tile = {"tile": t2, "ms_per_step": round(step2_ms, 4), "Mpoints_per_s": round(n / (step2_ms * 1e-3) / 1e6, 1),
                      "n_instances": int(counters2[1]), "n_tiles": int(layout2.n_tiles),
                      "max_abs_image_difference": float((image2 - image).abs().max())}
        del ws2, image2, alpha2, bw2, gf2, go2

    # the same points through the Gaussian footprint (the reference's other rasterizer mode), 8x8 tiles as in the
    # reference: a side measurement, not part of `value`
    gaussian = None
    try:
        if args.no_extras:
            raise RuntimeError("skipped (--no-extras)")
        gcfg = _lib.GaussianConfig(_lib.RasterConfig(n, 8, channels, _lib.FEAT_DIRECT_F32, 0,
                                                     _lib.make_camera(hv.camera)), 0.0, 3.0, 0, 0)
        glayout = _lib.GaussianLayout()
        _lib.check(lib.inpc_gaussian_layout_query(C.byref(gcfg), C.byref(glayout)), "gaussian layout")
        gws = torch.empty(glayout.total_bytes, dtype=torch.uint8, device=device)
        g_image, g_alpha, g_weights = torch.empty_like(image), torch.empty_like(alpha), torch.empty_like(blending_weights)
        g_gf, g_go = torch.empty_like(grad_features), torch.empty_like(grad_opacities)

        def gaussian_forward():
            _lib.check(lib.inpc_gaussian_forward(C.byref(gcfg), _lib.ptr(positions), _lib.ptr(features),
                                                 _lib.ptr(opacities), None, _lib.ptr(w2c), _lib.ptr(cam_position),
                                                 _lib.ptr(g_image), _lib.ptr(g_alpha), _lib.ptr(g_weights), None,
                                                 _lib.ptr(gws), glayout.total_bytes, stream), "inpc_gaussian_forward")

        def gaussian_backward():
            _lib.check(lib.inpc_gaussian_backward(C.byref(gcfg), _lib.ptr(grad_image), _lib.ptr(grad_alpha),
                                                  _lib.ptr(g_image), _lib.ptr(g_alpha), _lib.ptr(positions),
                                                  _lib.ptr(cam_position), _lib.ptr(g_gf), _lib.ptr(g_go), None,
                                                  _lib.ptr(gws), glayout.total_bytes, stream), "inpc_gaussian_backward")

        def gaussian_step():
            gaussian_forward()
            gaussian_backward()

        gaussian_step()
        g_counters = (C.c_uint32 * 4)()
        _lib.check(lib.inpc_gaussian_read_counters(C.byref(gcfg), _lib.ptr(gws), C.byref(g_counters), stream),
                   "inpc_gaussian_read_counters")
        g_step_ms = time_calls(gaussian_step, args.steps)
        g_fwd_ms = time_calls(gaussian_forward, args.steps)
        g_bwd_ms = time_calls(gaussian_backward, args.steps)
        with _lib.KernelTimer() as g_timer:
            for _ in range(args.steps):
                gaussian_step()
        g_kernels = {}
        for name, ms in g_timer.records:
            g_kernels[name] = g_kernels.get(name, 0.0) + ms / args.steps
        gaussian = {"workload": "same points, Gaussian footprint (training variance), 8x8 tiles, forward+backward",
                    "ms_per_step": round(g_step_ms, 4), "forward_ms": round(g_fwd_ms, 4),
                    "backward_ms": round(g_bwd_ms, 4), "Mpoints_per_s": round(n / (g_step_ms * 1e-3) / 1e6, 1),
                    "n_instances": int(g_counters[1]),
                    "kernel_ms_per_step": {k: round(v, 4) for k, v in sorted(g_kernels.items(), key=lambda kv: -kv[1])}}
        del gws, g_image, g_alpha, g_weights, g_gf, g_go
    except Exception as exc:  # the figure is optional
        print(f"bench.py: Gaussian footprint not measured: {exc}", file=sys.stderr)

    # the reference's own shape through the operator layer: (N,36) fp16 SH features -> 4 channels, autograd step
    # (forward + backward including the SH gradient), both footprints with the tile size the layer picks
    reference_shape = None
    try:
        if args.no_extras:
            raise RuntimeError("skipped (--no-extras)")
        from inpc_amd import INPCRasterizer

        sh = (torch.randn((n, 36), generator=gen, device=device) * 0.2).half().requires_grad_(True)
        op1 = opacities.reshape(n, 1).clone().requires_grad_(True)
        gi4 = torch.randn((4, H, W), generator=gen, device=device) * 1e-2
        rasterizer = INPCRasterizer()
        reference_shape = {}
        for mode_name, mode_value in (("bilinear", 0), ("gaussian", 1)):
            def api_step():
                sh.grad = None
                op1.grad = None
                img, alp, _ = rasterizer(view, mode_value, positions, sh, op1)
                torch.autograd.backward([img, alp], [gi4, grad_alpha])

            api_step()
            reference_shape[f"{mode_name}_ms_per_step"] = round(time_calls(api_step, max(args.steps // 2, 1)), 4)
        del sh, op1
    except Exception as exc:  # the figure is optional
        print(f"bench.py: reference-shaped step not measured: {exc}", file=sys.stderr)

    # BASELINE configuration 0, the reference's CPU-runnable case: forward only, 65,536 uniform points in the unit
    # cube, 4 fp32 channels ~U(0,1), opacity ~U(0.05,0.95), 256x256, f = 300, distance 3, 16x16 tiles, seed 0: the GPU
    # forward through the C ABI and the CPU oracle's forward on the same arrays
    config0 = None
    try:
        if args.no_extras:
            raise RuntimeError("skipped (--no-extras)")
        n0 = CONFIG0_POINTS
        hv0 = synthetic.camera_on_z(256, 256, 300.0, 3.0)
        view0 = hv0.to_view(device)
        pos0_h = synthetic.cube_points(n0, 1.0, 0)
        feats0_h, opac0_h = synthetic.point_attributes(n0, 4, "uniform", 0)
        pos0, feats0, opac0 = (torch.from_numpy(np.ascontiguousarray(a)).to(device) for a in (pos0_h, feats0_h, opac0_h))
        cfg0 = _lib.RasterConfig(n0, 16, 4, _lib.FEAT_DIRECT_F32, 0, _lib.make_camera(hv0.camera), 4 * n0)
        layout0 = _lib.RasterLayout()
        _lib.check(lib.inpc_raster_layout_query(C.byref(cfg0), C.byref(layout0)), "layout")
        ws0 = torch.empty(layout0.total_bytes, dtype=torch.uint8, device=device)
        image0 = torch.empty((4, 256, 256), dtype=torch.float32, device=device)
        alpha0 = torch.empty((1, 256, 256), dtype=torch.float32, device=device)
        bw0 = torch.empty(n0, dtype=torch.float32, device=device)
        w2c0, camp0 = view0.w2c.contiguous(), view0.position.contiguous()

        def forward0():
            _lib.check(lib.inpc_raster_forward(C.byref(cfg0), _lib.ptr(pos0), _lib.ptr(feats0), _lib.ptr(opac0),
                                               _lib.ptr(w2c0), _lib.ptr(camp0), _lib.ptr(image0), _lib.ptr(alpha0),
                                               _lib.ptr(bw0), None, _lib.ptr(ws0), layout0.total_bytes, stream),
                       "inpc_raster_forward")

        forward0()
        gpu0_ms = time_calls(forward0, 10 * args.steps)
        config0 = {"workload": f"{n0:,} pts uniform in the unit cube, 4 fp32 channels, 256x256, f=300, distance 3, "
                               "16x16 tiles, forward only",
                   "gpu_forward_ms": round(gpu0_ms, 4), "gpu_Mpoints_per_s": round(n0 / (gpu0_ms * 1e-3) / 1e6, 1)}
        if not args.no_cpu_baseline:
            from oracle import oracle as O

            c0 = hv0.camera
            ocfg0 = O.make_config(n0, O.make_camera(c0.width, c0.height, c0.focal_x, c0.focal_y, c0.center_x, c0.center_y,
                                                    c0.near_plane, c0.far_plane), 16, 4, O.FEAT_DIRECT_F32)
            ref0 = O.raster_forward(ocfg0, pos0_h, feats0_h, opac0_h, hv0.w2c)   # warm-up, and the images to compare
            config0["max_abs_image_difference_to_cpu"] = float(np.abs(image0.cpu().numpy() - ref0["image"]).max())
            threads0 = O.num_threads()
            for label, threads in (("cpu_forward_ms", threads0), ("cpu_single_thread_forward_ms", 1)):
                O.set_num_threads(threads)
                reps, spent = 0, 0.0
                while spent < 1.5 and reps < 200:
                    t = O.now()
                    O.raster_forward(ocfg0, pos0_h, feats0_h, opac0_h, hv0.w2c)
                    spent += O.now() - t
                    reps += 1
                config0[label] = round(spent * 1e3 / reps, 3)
            O.set_num_threads(threads0)
            config0["cpu_cores"] = threads0
        del ws0, image0, alpha0, bw0
    except Exception as exc:  # the figure is optional
        print(f"bench.py: configuration 0 not measured: {exc}", file=sys.stderr)

    # The reference's default inference frame: four times (expected-count samples for 8,388,352 requested points,
    # one sample per count, then the inference rasterizer on raw (N,37) fp16 appearance output), images added up.
    # The appearance network between the two is not part of this path: its output is random numbers made beforehand.
    inference_frame = None
    try:
        if args.no_extras:
            raise RuntimeError("skipped (--no-extras)")
        from inpc_amd import INPCRasterizer

        n_req, n_multi = FRAME_REQUESTED_SAMPLES, 4
        frame_sampler = ProbabilityFieldSampler(seed=0)
        probe = frame_sampler.generate_expected_samples(centers, levels, weights, view, n_req, 1, oct.initial_size)
        n_created = int(probe.shape[0])
        raw = (torch.randn((n_created, 37), generator=gen, device=device) * 0.5).half()
        frame_rasterizer = INPCRasterizer()
        del probe

        def frame():
            acc = None
            for _ in range(n_multi):
                p = frame_sampler.generate_expected_samples(centers, levels, weights, view, n_req, 1, oct.initial_size)
                img, dep, alp = frame_rasterizer.render(view, 0, p, raw[: p.shape[0]], 1.0, 3.0)
                if acc is None:
                    acc = [img, dep, alp]
                else:
                    acc[0] += img
                    acc[1] += dep
                    acc[2] += alp
            return acc

        frame()
        frame_ms = time_calls(frame, max(args.steps // 4, 2))
        with _lib.KernelTimer() as frame_timer:
            frame()
        frame_kernels = {}
        for name, ms in frame_timer.records:
            frame_kernels[name] = frame_kernels.get(name, 0.0) + ms
        inference_frame = {
            "workload": f"{n_multi} x (generate_expected_samples({n_req}, 1) -> {n_created} points, render on raw (N,37) "
                        f"fp16, bilinear footprint, 16x16 tiles) @{W}x{H}",
            "ms_per_frame": round(frame_ms, 3), "Mpoints_per_s": round(n_multi * n_created / (frame_ms * 1e-3) / 1e6, 1),
            "kernel_ms_per_frame": {k: round(v, 4) for k, v in sorted(frame_kernels.items(), key=lambda kv: -kv[1])}}
        del raw
    except Exception as exc:  # the figure is optional
        print(f"bench.py: inference frame not measured: {exc}", file=sys.stderr)

    # ---- per-kernel durations: HIP events around every launch, on the launch stream, same steps ----------
    with _lib.KernelTimer() as timer:
        for _ in range(args.steps):
            step()
    per_kernel = {}
    for name, ms in timer.records:
        tot, cnt = per_kernel.get(name, (0.0, 0))
        per_kernel[name] = (tot + ms, cnt + 1)
    pixels = H * W
    kernels = []
    for name, (tot, cnt) in sorted(per_kernel.items(), key=lambda kv: -kv[1][0]):
        avg_ms = tot / cnt
        launches = cnt / args.steps
        alg = algorithmic_bytes(name, n, n_visible, n_instances, pixels, channels, layout.end_bit) / launches
        kernels.append({"kernel": name, "launches_per_step": launches, "avg_ms": round(avg_ms, 5),
                        "ms_per_step": round(tot / args.steps, 5),
                        "algorithmic_GBps": round(alg / (avg_ms * 1e-3) / 1e9, 1) if alg > 0 and avg_ms > 0 else None})
    dominant = kernels[0]
    dom_alg = algorithmic_bytes(dominant["kernel"], n, n_visible, n_instances, pixels, channels, layout.end_bit) \
        / dominant["launches_per_step"]
    achieved = dom_alg / (dominant["avg_ms"] * 1e-3) / 1e9
    traffic = measured_traffic(dominant["kernel"], args.workload)
    roofline = {"bound": "hbm", "kernel": dominant["kernel"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_source": None if traffic is None else
                f"{traffic_file(args.workload).relative_to(ROOT)} (profiler counters of an earlier run of this "
                "command, not measured by this run)",
                "algorithmic_bytes_per_launch": dom_alg, "avg_launch_ms": dominant["avg_ms"]}
    fwd_bytes, bwd_bytes = step_algorithmic_bytes(n, n_visible, n_instances, pixels, channels, layout.end_bit)
    step_gbps = (fwd_bytes + bwd_bytes) / (ms_per_step * 1e-3) / 1e9

    # ---- CPU baseline: the oracle on a bounded sample of the same workload --------------------------------
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import oracle as O

        n_cpu = min(n, 1_048_576)
        c = hv.camera
        cam = O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane,
                            c.far_plane)
        ocfg = O.make_config(n_cpu, cam, tile, channels, O.FEAT_DIRECT_F32)
        pos_h = positions[:n_cpu].cpu().numpy()
        feat_h = features[:n_cpu].cpu().numpy()
        opac_h = opacities[:n_cpu].cpu().numpy()
        gi_h, ga_h = grad_image.cpu().numpy(), grad_alpha.cpu().numpy()
        O.raster_forward_backward(ocfg, pos_h, feat_h, opac_h, hv.w2c, gi_h, ga_h)  # warm-up

        def cpu_leg(seconds):
            reps, spent = 0, 0.0
            while spent < seconds and reps < 1000:
                t = O.now()
                O.raster_forward_backward(ocfg, pos_h, feat_h, opac_h, hv.w2c, gi_h, ga_h)
                spent += O.now() - t
                reps += 1
            return reps, spent

        all_threads = O.num_threads()
        reps, spent = cpu_leg(args.cpu_seconds)
        O.set_num_threads(1)
        reps1, spent1 = cpu_leg(args.cpu_seconds / 2)
        O.set_num_threads(all_threads)
        cpu = {"value": round(n_cpu * reps / spent / 1e6, 3), "unit": "Mpoints/s", "cores": all_threads,
               "kind": "port",
               "sample": f"first {n_cpu} of the {n} points, same camera/image/channels/tiles, forward+backward, "
                         f"{reps} repetitions, {spent:.1f} s",
               "single_thread": {"value": round(n_cpu * reps1 / spent1 / 1e6, 3), "unit": "Mpoints/s", "cores": 1,
                                 "sample": f"same sample, {reps1} repetitions, {spent1:.1f} s"}}

    config4 = None
    if not args.no_config4 and not args.no_extras and args.workload.startswith("config3"):
        # free the training workload first: this one needs about 12 GB
        del workspace, image, alpha, blending_weights, grad_features, grad_opacities, features, opacities
        torch.cuda.empty_cache()
        config4 = config4_leg()

    # the sampler (training draw of the same n points): 32 B per leaf (20 in, 4 out, 8 scan) and 32 B per candidate
    # (16 B of leaf data gathered, 12 B position + 4 B index written); the CDF probes are cache traffic and not counted
    draw_kernel_ms = sum(draw_kernels.values())
    draw_bytes = 32.0 * wl["leaves"] + 32.0 * draw_candidates
    sampler_extra = {
        "workload": f"training draw of {n} samples from {wl['leaves']} leaves (level {wl['level']}), same camera",
        "call_ms": round(sampler_ms, 3), "kernels_ms": round(draw_kernel_ms, 4), "launches": len(draw_timer.records),
        "candidates": draw_candidates,
        "Msamples_per_s": round(n / (sampler_ms * 1e-3) / 1e6, 1),
        "Msamples_per_s_kernels_only": round(n / (draw_kernel_ms * 1e-3) / 1e6, 1) if draw_kernel_ms > 0 else None,
        "algorithmic_bytes": draw_bytes,
        "algorithmic_GBps": round(draw_bytes / (draw_kernel_ms * 1e-3) / 1e9, 1) if draw_kernel_ms > 0 else None,
        "hbm_frac": round(draw_bytes / (draw_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if draw_kernel_ms > 0 else None,
        "kernel_ms": {k: round(v, 4) for k, v in sorted(draw_kernels.items(), key=lambda kv: -kv[1])},
    }

    out = {
        "metric": "Mpoints/s, rasterizer fwd+bwd, 8M pts @1237x822 (ms/frame in ms_per_step)",
        "value": round(n / (ms_per_step * 1e-3) / 1e6, 2),
        "unit": "Mpoints/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": wl["describe"], "n_points": n, "n_visible": n_visible, "n_instances": n_instances,
                   "image": [W, H], "channels": channels, "tile": tile},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": {
            "forward_ms": round(fwd_ms, 4), "backward_ms": round(bwd_ms, 4),
            "graph_replay_ms": None if graph_ms is None else round(graph_ms, 4),
            "sampler": sampler_extra,
            "field_update_ms": None if field_ms is None else round(field_ms, 4),
            "other_tile_size": other_tile,
            "gaussian_footprint": gaussian,
            "sh36_autograd_step": reference_shape,
            "config0": config0,
            "inference_frame": inference_frame,
            "config4_inference": config4,
            "step_algorithmic_GB": round((fwd_bytes + bwd_bytes) / 1e9, 3),
            "step_algorithmic_GBps": round(step_gbps, 1), "step_hbm_frac": round(step_gbps / HBM_PEAK_GBS, 4),
            "kernels": kernels,
        },
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
