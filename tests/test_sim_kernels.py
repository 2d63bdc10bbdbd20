"""The library's kernels on the CPU: a selection of the GPU parity tests, run without a GPU.

tests/cpu_sim compiles inpc_amd/csrc/*.hip unchanged for the host against a stand-in for the HIP runtime in which the
threads of a block are fibers and a wave's ballots, shuffles, DPP moves and barriers are meeting points. Each case
below is a test function of one of the GPU test modules, called with the simulator's library loaded in the HIP
library's place and host memory as the device: the same C-ABI calls, the same oracle, the same tolerances. The cases
are chosen to finish in about two minutes together and to reach every kernel; `pytest tests -m gpu --sim` runs all
of the GPU tests this way (about forty minutes, most of it the full-size configurations of test_gpu_full_size.py).

INPC_SIM_ORDER=reverse or =shuffle in the environment makes the simulator resume the threads of a block (and the
blocks of a grid) in another order: a kernel whose lanes hand data to each other without a barrier, or that relies on
the order of its blocks, then gives other results; all cases pass under all three orders.

This shows the kernels' indexing, arithmetic and synchronisation right or wrong. It says nothing about speed and
nothing about what only the hardware does (scheduling of blocks against each other, memory ordering between blocks,
register and LDS limits): the `gpu` tests stay the parity tests proper."""
import importlib
import inspect
import os
import subprocess
import sys
from pathlib import Path

import pytest

CASES = [
    # ---- sampler: leaf weights, CDF, draws (all bit-exact)
    ("test_gpu_sampler", "test_leaf_weights_and_cdf_bit_exact", dict(n_leaves=65, level=4)),
    ("test_gpu_sampler", "test_leaf_weights_and_cdf_bit_exact", dict(n_leaves=6000, level=6)),
    ("test_gpu_sampler", "test_leaf_weights_and_cdf_bit_exact", dict(n_leaves=300000, level=8)),
    ("test_gpu_sampler", "test_cdf_and_search_tree_against_their_definitions", dict(n_leaves=2)),
    ("test_gpu_sampler", "test_cdf_and_search_tree_against_their_definitions", dict(n_leaves=16384)),
    ("test_gpu_sampler", "test_cdf_and_search_tree_against_their_definitions", dict(n_leaves=278528)),
    ("test_gpu_sampler", "test_cdf_and_search_tree_against_their_definitions", dict(n_leaves=4194304 + 65)),
    ("test_gpu_sampler", "test_cdf_of_exact_integers_matches_cumsum", {}),
    ("test_gpu_sampler", "test_sum_not_positive_leaves_weights_untouched", {}),
    ("test_gpu_sampler", "test_sample_bit_exact_and_stream_continues", dict(n_samples=2049)),
    ("test_gpu_sampler", "test_sample_bit_exact_and_stream_continues", dict(n_samples=100000)),
    ("test_gpu_sampler", "test_sample_bit_exact_across_octree_sizes", dict(n_leaves=17, level=3)),
    ("test_gpu_sampler", "test_sample_bit_exact_across_octree_sizes", dict(n_leaves=278528, level=9)),
    ("test_gpu_sampler", "test_sample_failure_path_writes_nothing", {}),
    ("test_gpu_sampler", "test_cull_compact_rounds_bit_exact", dict(rounds=[2048, 2047, 1, 30000], ids_int64=False)),
    ("test_gpu_sampler", "test_cull_compact_rounds_bit_exact", dict(rounds=[10000, 10000, 10000], ids_int64=True)),
    ("test_gpu_sampler", "test_training_api_matches_oracle_draw", {}),
    ("test_gpu_sampler", "test_training_api_draw_of_several_rounds", {}),
    ("test_gpu_sampler", "test_training_api_failure_pattern", {}),
    ("test_gpu_sampler", "test_generate_samples_and_expected_samples_api", {}),
    ("test_gpu_sampler", "test_expected_counts_without_a_positive_sum_are_all_zero", {}),
    ("test_gpu_sampler", "test_training_draw_that_never_hits_the_frustum_is_filled_with_the_failure_pattern", {}),
    # ---- bilinear rasterizer
    ("test_gpu_raster", "test_forward_direct_f32", dict(tile=8, channels=4)),
    ("test_gpu_raster", "test_forward_direct_f32", dict(tile=16, channels=8)),
    ("test_gpu_raster", "test_forward_direct_f32", dict(tile=8, channels=16)),
    ("test_gpu_raster", "test_forward_dense_opaque_scene_terminates_early", dict(tile=16)),
    ("test_gpu_raster", "test_forward_sh36_and_backward", dict(tile=8)),
    ("test_gpu_raster", "test_forward_sh36_and_backward", dict(tile=16)),
    ("test_gpu_raster", "test_backward_direct", dict(tile=16, channels=8, mode="f32")),
    ("test_gpu_raster", "test_backward_direct", dict(tile=8, channels=4, mode="f32")),
    ("test_gpu_raster", "test_backward_direct", dict(tile=16, channels=16, mode="f32")),
    ("test_gpu_raster", "test_backward_direct", dict(tile=8, channels=8, mode="f16")),
    ("test_gpu_raster", "test_inference_raw37_and_preextracted", dict(tile=16)),
    ("test_gpu_raster", "test_inference_direct_f16_16_channels", {}),
    ("test_gpu_raster", "test_edge_cases", dict(tile=8)),
    ("test_gpu_raster", "test_edge_cases", dict(tile=16)),
    ("test_gpu_raster", "test_non_finite_and_extreme_positions",
     dict(seed=70002, n=2000, width=37, height=211, tile=16, channels=4)),
    ("test_gpu_raster", "test_runs_of_equal_depth_keys", dict(tile=16, levels=400)),
    ("test_gpu_raster", "test_runs_of_equal_depth_keys", dict(tile=8, levels=30)),
    ("test_gpu_raster", "test_instances_beyond_the_capacity_are_reported_and_nothing_is_drawn", {}),
    ("test_gpu_raster", "test_operator_layer_grows_the_workspace_when_the_default_capacity_is_exceeded", {}),
    ("test_gpu_raster", "test_autograd_api_sh_and_direct", {}),
    ("test_gpu_raster", "test_backward_twice_after_one_forward", dict(tile=16)),
    ("test_gpu_raster", "test_random_scenes_forward_backward", dict(case=101)),
    ("test_gpu_raster", "test_random_scenes_forward_backward", dict(case=103)),
    ("test_gpu_raster", "test_random_scenes_forward_backward", dict(case=105)),
    # ---- Gaussian footprint
    ("test_gpu_gaussian", "test_forward_direct_f32", dict(tile=16, channels=4)),
    ("test_gpu_gaussian", "test_forward_direct_f32", dict(tile=8, channels=8)),
    ("test_gpu_gaussian", "test_forward_backward_dense_opaque_scene", dict(tile=16)),
    ("test_gpu_gaussian", "test_forward_sh36_and_backward", dict(tile=8)),
    ("test_gpu_gaussian", "test_backward_direct", dict(mode="f16")),
    ("test_gpu_gaussian", "test_backward_direct", dict(mode="f32")),
    ("test_gpu_gaussian", "test_inference_preextracted", dict(tile=16, with_scales=True)),
    ("test_gpu_gaussian", "test_inference_raw37", {}),
    ("test_gpu_gaussian", "test_edge_cases", {}),
    ("test_gpu_gaussian", "test_non_finite_and_extreme_positions", dict(seed=71002, n=2000, width=37, height=211, tile=16)),
    ("test_gpu_gaussian", "test_instances_beyond_the_capacity_are_reported", {}),
    ("test_gpu_gaussian", "test_random_scenes_forward_backward", dict(case=201)),
    ("test_gpu_gaussian", "test_random_scenes_forward_backward", dict(case=205)),   # footprints of hundreds of pixels
    # ---- probability field bookkeeping, element-wise operators, the reference's module names
    ("test_gpu_field", "test_update_bit_exact", dict(n_leaves=1000, n_samples=257)),
    ("test_gpu_field", "test_two_updates_in_a_row_and_bad_index", {}),
    ("test_gpu_field", "test_closes_the_loop_with_sampler_and_rasterizer", {}),
    ("test_gpu_field", "test_prune_bit_exact", dict(n=70001)),
    ("test_gpu_field", "test_prune_everything_and_nothing", {}),
    ("test_gpu_field", "test_subdivide_bit_exact", dict(n=33333)),
    ("test_gpu_field", "test_extract_global_bit_exact", {}),
    ("test_gpu_field", "test_morton_codes_bit_exact_and_the_ordered_extraction", {}),
    ("test_gpu_misc", "test_spherical_contraction", {}),
    ("test_gpu_misc", "test_feature_to_opacity_forward_and_backward", {}),
    ("test_gpu_misc", "test_weight_decay_grads", {}),
    ("test_gpu_misc", "test_fused_cauchy_loss", {}),
    ("test_gpu_c_module", "test_training_pass_with_the_reference_call_pattern", dict(mode="BILINEAR")),
    ("test_gpu_c_module", "test_inference_calls", dict(mode="GAUSSIAN")),
    ("test_gpu_c_module", "test_sampler_class_and_viewpoint_weights", {}),
    ("test_gpu_c_module", "test_elementwise_functions", {}),
    # ---- the entry point that allocates nothing
    ("test_zz_no_alloc", "test_static_scratch_matches_workspace_variant_on_two_calls_in_a_row", {}),
    ("test_zz_no_alloc", "test_static_scratch_rejects_sizes_beyond_its_maximum_and_short_heads", {}),
    # ---- the committed fixtures
    ("test_golden", "test_hip_sampler_gives_fixture", {}),
    ("test_golden", "test_hip_rasterizer_gives_fixture", {}),
    ("test_golden", "test_hip_gaussian_footprint_gives_fixture", {}),
]


def _case_id(case):
    module, name, kwargs = case
    tail = "-".join(str(v).replace(" ", "") for v in kwargs.values())
    return f"{module[5:]}.{name[5:]}" + (f"[{tail}]" if tail else "")


def _resolve(module, kwargs):
    """Spelled-out values for the parameters that the GPU modules take as objects."""
    out = dict(kwargs)
    if "case" in out:   # a row of the module's RANDOM_CASES, named by its seed
        out["case"] = next(c for c in module.RANDOM_CASES if c[0] == out["case"])
    if isinstance(out.get("mode"), str) and hasattr(module, "RasterizerMode"):
        out["mode"] = getattr(module.RasterizerMode, out["mode"])
    return out


@pytest.mark.parametrize("case", CASES, ids=_case_id)
def test_on_the_simulator(sim, oracle, request, case):
    module_name, name, kwargs = case
    module = importlib.import_module(f"tests.{module_name}")
    function = getattr(module, name)
    arguments = _resolve(module, kwargs)
    for parameter in inspect.signature(function).parameters:
        if parameter == "gpu":
            arguments[parameter] = sim
        elif parameter == "oracle":
            arguments[parameter] = oracle
        elif parameter not in arguments:
            arguments[parameter] = request.getfixturevalue(parameter)   # monkeypatch, a module's own fixtures
    function(**arguments)


def test_every_case_names_a_gpu_test():
    """The selection above cannot rot: every entry is a collected test of its module, with parameters it takes."""
    for module_name, name, kwargs in CASES:
        module = importlib.import_module(f"tests.{module_name}")
        function = getattr(module, name)
        taken = set(inspect.signature(function).parameters)
        assert set(kwargs) <= taken, (module_name, name, kwargs)
        marks = [m.name for m in getattr(function, "pytestmark", [])]
        assert "real_gpu" not in marks, (module_name, name)


@pytest.mark.parametrize("order", ["reverse", "shuffle"])
def test_results_do_not_depend_on_the_order_of_threads_and_blocks(order):
    """A handful of the cases above in a process of their own whose simulator resumes threads and blocks in another
    order (the order is fixed when the library is loaded): gradient rows of straddling points, ties in the tile sort,
    large Gaussian footprints, the CDF, the ordered compaction of the training draw."""
    chosen = ("gpu_raster.backward_direct[16-8-f32]", "gpu_raster.runs_of_equal_depth_keys[8-30]",
              "gpu_gaussian.random_scenes_forward_backward[205]",
              "gpu_sampler.cdf_and_search_tree_against_their_definitions[278528]",
              "gpu_sampler.cull_compact_rounds_bit_exact[[10000,10000,10000]-True]",
              "gpu_field.closes_the_loop_with_sampler_and_rasterizer")
    nodes = [f"{Path(__file__)}::test_on_the_simulator[{case}]" for case in chosen]
    env = dict(os.environ, INPC_SIM_ORDER=order)
    done = subprocess.run([sys.executable, "-m", "pytest", *nodes, "-q", "-x", "-p", "no:cacheprovider"], env=env,
                          capture_output=True, text=True, stdin=subprocess.DEVNULL, timeout=900,
                          cwd=Path(__file__).resolve().parent.parent)
    assert done.returncode == 0, done.stdout[-3000:] + done.stderr[-2000:]
    assert f"{len(chosen)} passed" in done.stdout, done.stdout[-2000:]


def test_images_and_gradients_are_the_same_bits_under_any_order(tmp_path):
    """One scene through both footprints under three orders of threads and blocks (and three byte patterns in the LDS
    that a block finds): images, alphas and both gradients come out bit for bit the same (their sums have a fixed order: no float atomics), which no run on the hardware can
    show; only the blending weights of points that straddle tiles are added up by float atomics, as in the reference
    (B/rasterization/src/bilinear/kernels.cu:294; the reference adds its gradients that way too, :399-402), and may differ in
    the last bit."""
    import numpy as np

    probe = Path(__file__).resolve().parent / "cpu_sim" / "order_probe.py"
    runs = {}
    for order, lds_byte in (("forward", "0xCD"), ("reverse", "0x00"), ("shuffle", "0xFF")):   # and what LDS holds at first
        out = tmp_path / f"{order}.npz"
        runs[order] = (out, subprocess.Popen([sys.executable, str(probe), str(out)],
                                            env=dict(os.environ, INPC_SIM_ORDER=order, INPC_SIM_LDS_BYTE=lds_byte),
                                            stdin=subprocess.DEVNULL, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
    results = {}
    for order, (out, process) in runs.items():
        log, _ = process.communicate(timeout=900)
        assert process.returncode == 0, log[-3000:]
        results[order] = np.load(out)
    base = results["forward"]
    assert len(base.files) == 20
    for order in ("reverse", "shuffle"):
        for name in base.files:
            a, b = base[name], results[order][name]
            if name.endswith("blending_weights"):
                np.testing.assert_allclose(a, b, rtol=0, atol=2e-7, err_msg=f"{name} under {order}")
            else:
                np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32), err_msg=f"{name} under {order}")
