"""bench.py and __graft_entry__.smoke() from end to end without a GPU. Every leg of the benchmark (the timed step, the
roofline and CPU-baseline objects, the sampler draw, the other tile size, the Gaussian footprint, the reference-shaped autograd step, configuration 0, the
inference frame, configuration 4) runs once on shrunken sizes through the kernels compiled for the CPU simulator of
tests/cpu_sim, with a stand-in for the few torch.cuda calls the script makes. The figures mean nothing here (the
simulator is thousands of times slower than the device); what is checked is that the script runs, prints its one JSON
line with the fields the benchmark contract names, and that no optional leg has silently dropped out."""
import contextlib
import importlib.util
import json
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


class _Stream:
    def synchronize(self):
        pass


class _NoGraph:
    def __init__(self):
        raise RuntimeError("graphs need the device")


@pytest.fixture
def bench_on_the_simulator(sim, monkeypatch):
    spec = importlib.util.spec_from_file_location("bench_dry_run", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    monkeypatch.setattr(bench, "DEVICE", "cpu")
    monkeypatch.setattr(bench, "CONFIG0_POINTS", 3_000)
    monkeypatch.setattr(bench, "FRAME_REQUESTED_SAMPLES", 8_000)
    monkeypatch.setattr(bench, "CONFIG4", dict(n=12_000, width=123, height=82, focal=100.0, leaves=70_000, level=8))
    monkeypatch.setitem(bench.WORKLOADS, "config3", dict(n=10_000, width=160, height=100, focal=125.0, channels=8,
                                                         tile=16, leaves=5000, level=6, describe="dry run"))
    for name, value in dict(is_available=lambda: True, set_device=lambda d: None, synchronize=lambda *a: None,
                            empty_cache=lambda: None, Stream=_Stream, stream=lambda s: contextlib.nullcontext(),
                            CUDAGraph=_NoGraph).items():
        monkeypatch.setattr(torch.cuda, name, value)
    # the script allocates its workspaces itself; the device's allocator aligns to 256 bytes, the host's does not
    real_empty = torch.empty

    def aligned_empty(*size, **kw):
        if kw.get("dtype") is torch.uint8 and len(size) == 1 and isinstance(size[0], int):
            raw = real_empty(size[0] + 256, **kw)
            skip = (-raw.data_ptr()) % 256
            return raw[skip:skip + size[0]]
        return real_empty(*size, **kw)

    monkeypatch.setattr(torch, "empty", aligned_empty)
    return bench


def test_every_leg_of_the_benchmark_runs(bench_on_the_simulator, monkeypatch, capsys):
    monkeypatch.setattr(sys, "argv", ["bench.py", "--steps", "1", "--warmup", "1", "--cpu-seconds", "0.2"])
    assert bench_on_the_simulator.main() == 0
    out = capsys.readouterr()
    lines = [line for line in out.out.splitlines() if line.startswith("{")]
    assert len(lines) == 1, out.out
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 1 and record["warmup"] == 1
    assert record["vs_baseline"] is None and record["dtype"] == "f32" and record["data"] == "synthetic"
    assert set(record["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert record["roofline"]["bound"] == "hbm" and record["roofline"]["peak"] == 8000.0
    assert set(record["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    extra = record["extra"]
    # every optional leg delivered its figure (only the graph replay cannot: it needs the device)
    for key in ("forward_ms", "backward_ms", "sampler", "field_update_ms", "other_tile_size", "gaussian_footprint",
                "sh36_autograd_step", "config0", "inference_frame", "config4_inference", "kernels"):
        assert extra.get(key) is not None, (key, out.err)
    assert extra["graph_replay_ms"] is None
    assert extra["config0"]["max_abs_image_difference_to_cpu"] < 1e-5
    assert extra["other_tile_size"]["max_abs_image_difference"] < 1e-5
    assert extra["config4_inference"]["bilinear_abi"]["roofline"]["kernel"]
    assert {"sample_cull_compact", "cdf_tile_totals", "cdf_scan_tiles", "cdf_finish"} <= set(extra["sampler"]["kernel_ms"])
    # a training draw that needs one round: leaf weights, three for the CDF, the round's reset, the draw, its end
    assert extra["sampler"]["launches"] == 7


def test_the_large_frame_alone(bench_on_the_simulator, monkeypatch, capsys):
    monkeypatch.setattr(sys, "argv", ["bench.py", "--only-config4"])
    assert bench_on_the_simulator.main() == 0
    out = capsys.readouterr()
    lines = [line for line in out.out.splitlines() if line.startswith("{")]
    assert len(lines) == 1, out.out
    record = json.loads(lines[0])
    assert record["roofline"]["kernel"].startswith("raster_") and record["cpu_baseline"] is None
    assert record["extra"]["config4_inference"]["bilinear_abi"]["n_visible"] > 0
    assert record["config"]["workload"].startswith("12,000 pts")


def test_smoke_runs(sim, monkeypatch, capsys):
    """__graft_entry__.smoke(), the check that runs on the GPU box before the benchmark, through the simulator."""
    spec = importlib.util.spec_from_file_location("graft_entry_dry_run", ROOT / "__graft_entry__.py")
    entry = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(entry)
    monkeypatch.setattr(entry, "SMOKE_DEVICE", "cpu")
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    entry.smoke()
    assert "smoke ok" in capsys.readouterr().out


def test_more_than_one_gpu_is_refused(monkeypatch, capsys):
    spec = importlib.util.spec_from_file_location("bench_refusal", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    monkeypatch.setattr(sys, "argv", ["bench.py", "--gpus", "2"])
    assert bench.main() == 2
    assert "one GPU" in capsys.readouterr().err
