"""GPU parity of the sampler against the CPU oracle, through the C ABI. Leaf weights, CDF, leaf ids,
positions, cull decisions and the generator state must be bit-exact."""
import ctypes as C

import numpy as np
import pytest
import torch

from inpc_amd import _lib, synthetic
from tests import helpers as H

pytestmark = pytest.mark.gpu


def small_scene(n_leaves=6000, level=6, seed=3, mixed_levels=True, distance=3.5):
    oct = synthetic.octree_leaves(n_leaves, level, initial_size=4.0, seed=seed)
    if mixed_levels:  # leaves of several sizes (geometry need not tile space for the sampler)
        rng = np.random.default_rng(seed + 100)
        oct.levels = rng.integers(3, 9, size=n_leaves).astype(np.int32)
    hv = synthetic.camera_on_z(311, 203, 260.0, distance)
    return oct, hv


def oracle_cam(O, hv):
    c = hv.camera
    return O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)


@pytest.mark.parametrize("n_leaves,level", [(1, 0), (63, 4), (64, 4), (65, 4), (4097, 5), (6000, 6), (300000, 8)])
def test_leaf_weights_and_cdf_bit_exact(gpu, oracle, n_leaves, level):
    oct, hv = small_scene(n_leaves, level, mixed_levels=n_leaves > 100)
    w_gpu = H.leaf_weights(oct, hv)
    w_ref = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, oracle_cam(oracle, hv), oct.initial_size)
    np.testing.assert_array_equal(w_gpu.cpu().numpy().view(np.uint32), w_ref.view(np.uint32))
    cdf_gpu, total_gpu = H.build_cdf(w_gpu)
    ok, cdf_ref, total_ref = oracle.build_cdf(w_ref)
    assert ok
    assert total_gpu.cpu().numpy().view(np.uint32)[0] == np.float32(total_ref).view(np.uint32)
    np.testing.assert_array_equal(cdf_gpu.cpu().numpy().view(np.uint32), cdf_ref.view(np.uint32))


def test_cdf_of_exact_integers_matches_cumsum(gpu):
    # Integer-valued weights whose total is a power of two: the total, the reciprocal, the normalised
    # weights and every partial sum are exact in fp32 whatever the association order, so the CDF must
    # equal numpy's cumsum bit for bit. Pins chunk indexing (dropped / doubled elements) without the oracle.
    rng = np.random.default_rng(0)
    n = 70001
    w = rng.integers(0, 8, size=n).astype(np.int64)
    w[-1] += (1 << 18) - w.sum()
    assert 0 <= w[-1] < (1 << 18)
    cdf, tot = H.build_cdf(H.dev(w.astype(np.float32)))
    assert float(tot[0].item()) == float(1 << 18)
    expect = (np.cumsum(w).astype(np.float64) / (1 << 18)).astype(np.float32)
    np.testing.assert_array_equal(cdf.cpu().numpy(), expect)


def search_tree_of(cdf, n_nodes):
    """The head of a CDF as the probe sequence of B/sampling/include/sampling_utils.h:49-69 defines it: node 1 is the
    element the first probe reads, nodes 2k and 2k + 1 those of the probe after going left and right; 0 where a
    search has ended before."""
    n = len(cdf)
    head = np.zeros(n_nodes, np.float32)
    first, count = np.zeros(1, np.int64), np.full(1, n, np.int64)
    depth = 0
    while (1 << depth) < n_nodes:
        nodes = (1 << depth) + np.arange(1 << depth)
        live = count > 0
        head[nodes[live]] = cdf[first[live] + count[live] // 2]
        step = count // 2
        left_first, left_count = first, np.where(live, step, 0)
        right_first, right_count = first + step + 1, np.where(live, count - step - 1, 0)
        first = np.stack([left_first, right_first], 1).reshape(-1)
        count = np.stack([left_count, right_count], 1).reshape(-1)
        depth += 1
    return head


@pytest.mark.parametrize("n_leaves", [1, 2, 100, 16383, 16384, 70001, 278528, 4194304 + 65, 16777216 + 4097],
                         ids=lambda n: f"{n}leaves")
def test_cdf_and_search_tree_against_their_definitions(gpu, oracle, n_leaves):
    # the CDF against the oracle and the head against the probe sequence replayed on the indices, for octrees whose
    # tile totals fill one chunk, several chunks (above 262,144 leaves) and more than 4096 (above 16,777,216 leaves:
    # one more level of totals)
    rng = np.random.default_rng(n_leaves)
    w = np.exp(rng.normal(0.0, 1.0, size=n_leaves)).astype(np.float32)
    w[rng.random(n_leaves) < 0.25] = 0.0
    w[0] = 1.0
    cdf, head = H.build_cdf(H.dev(w))
    ok, cdf_ref, total_ref = oracle.build_cdf(w)
    assert ok
    cdf, head = cdf.cpu().numpy(), head.cpu().numpy()
    np.testing.assert_array_equal(cdf.view(np.uint32), cdf_ref.view(np.uint32))
    assert head[:1].view(np.uint32)[0] == np.float32(total_ref).view(np.uint32)
    want = search_tree_of(cdf_ref, len(head))
    np.testing.assert_array_equal(head[1:].view(np.uint32), want[1:].view(np.uint32))


def test_sum_not_positive_leaves_weights_untouched(gpu):
    w = np.zeros(5000, dtype=np.float32)
    cdf, total = H.build_cdf(H.dev(w))
    assert float(total[0].item()) == 0.0
    np.testing.assert_array_equal(cdf.cpu().numpy(), w)


@pytest.mark.parametrize("n_samples", [1, 255, 2048, 2049, 100000])
def test_sample_bit_exact_and_stream_continues(gpu, oracle, n_samples):
    oct, hv = small_scene()
    w = H.leaf_weights(oct, hv)
    cdf, total = H.build_cdf(w)
    rng_dev = H.make_rng(1234)
    rng_ref = oracle.Pcg32(1234)
    cdf_host = cdf.cpu().numpy()
    for _ in range(2):  # the second call must continue the generator stream
        pos, ids = H.sample(oct, cdf, total, n_samples, rng_dev)
        pos_ref, ids_ref = oracle.sample(oct.centers, oct.levels, cdf_host, n_samples, oct.initial_size, rng_ref)
        np.testing.assert_array_equal(ids, ids_ref)
        np.testing.assert_array_equal(pos.view(np.uint32), pos_ref.view(np.uint32))
        assert H.rng_values(rng_dev) == (int(rng_ref.state[0]), int(rng_ref.state[1]))


@pytest.mark.parametrize("n_leaves,level", [(15, 3), (16, 3), (17, 3), (262144, 9), (278527, 9), (278528, 9),
                                            (300001, 9), (1048576, 10), (1500003, 11)])
def test_sample_bit_exact_across_octree_sizes(gpu, oracle, n_leaves, level):
    # The searches end in three ways: probes to the last element (fewer than 16 leaves), the last 16 elements fetched
    # by four lanes (up to 278,527 leaves), and further tree levels read from memory in front of that (more leaves;
    # sizes that are not powers of two leave the tree with ranges that do not start at multiples of 16). Many equal CDF
    # elements (leaves outside the frustum weigh nothing), elements an ulp above their successor (where a chunk of the
    # blocked scan ends) and samples at both ends of the CDF come with the scene.
    oct, hv = small_scene(n_leaves, level, seed=5, mixed_levels=False, distance=1.5)
    w = H.leaf_weights(oct, hv)
    cdf, total = H.build_cdf(w)
    cdf_host = cdf.cpu().numpy()
    assert n_leaves < 1000 or (np.diff(cdf_host) == 0).mean() > 0.05
    assert n_leaves < 200000 or (np.diff(cdf_host) < 0).any()
    rng_dev, rng_ref = H.make_rng(77), oracle.Pcg32(77)
    n_samples = 150000
    pos, ids = H.sample(oct, cdf, total, n_samples, rng_dev)
    pos_ref, ids_ref = oracle.sample(oct.centers, oct.levels, cdf_host, n_samples, oct.initial_size, rng_ref)
    np.testing.assert_array_equal(ids, ids_ref)
    np.testing.assert_array_equal(pos.view(np.uint32), pos_ref.view(np.uint32))
    # the training draw takes the same path through the cull kernel
    draw = H.CullDraw(oct, hv, cdf, total, rng_dev, 100000, 100000)
    acc, cons = draw.round(100000)
    pos_ref, ids_ref, acc_ref, cons_ref = oracle.sample_cull_compact(
        oct.centers, oct.levels, cdf_host, hv.w2c, oracle_cam(oracle, hv), oct.initial_size, rng_ref, 100000, 0, 100000)
    assert (acc, cons) == (acc_ref, cons_ref) and 0 < acc
    np.testing.assert_array_equal(draw.ids.cpu().numpy()[:acc], ids_ref[:acc])
    np.testing.assert_array_equal(draw.pos.cpu().numpy()[:acc].view(np.uint32), pos_ref[:acc].view(np.uint32))


def test_sample_failure_path_writes_nothing(gpu):
    oct, hv = small_scene(500, 4)
    w = torch.zeros(500, dtype=torch.float32, device=gpu)
    cdf, total = H.build_cdf(w)
    rng_dev = H.make_rng(5)
    before = H.rng_values(rng_dev)
    pos, ids = H.sample(oct, cdf, total, 1000, rng_dev)
    assert np.isnan(pos).all() and (ids == -7).all()
    assert H.rng_values(rng_dev) == before


@pytest.mark.parametrize("ids_int64", [False, True], ids=["int32_ids", "int64_ids"])
@pytest.mark.parametrize("rounds", [[50000], [2048, 2047, 1, 30000], [10000, 10000, 10000]])
def test_cull_compact_rounds_bit_exact(gpu, oracle, rounds, ids_int64):
    oct, hv = small_scene(distance=2.2)  # close camera: a good share of candidates is rejected
    cam = oracle_cam(oracle, hv)
    w = H.leaf_weights(oct, hv)
    cdf, total = H.build_cdf(w)
    cdf_host = cdf.cpu().numpy()
    capacity = 20000
    rng_dev = H.make_rng(77)
    rng_ref = oracle.Pcg32(77)
    draw = H.CullDraw(oct, hv, cdf, total, rng_dev, capacity, max(rounds), ids_int64=ids_int64)
    pos_ref, ids_ref, acc_ref, cons_ref, k0 = None, None, 0, 0, 0
    for m in rounds:
        acc_gpu, cons_gpu = draw.round(m)
        pos_ref, ids_ref, acc_ref, c = oracle.sample_cull_compact(oct.centers, oct.levels, cdf_host, hv.w2c, cam,
                                                                  oct.initial_size, rng_ref, capacity, k0, m, pos_ref,
                                                                  ids_ref, acc_ref)
        cons_ref = c or cons_ref
        k0 += m
        assert cons_gpu == cons_ref
        if cons_ref == 0:
            assert acc_gpu == acc_ref
        else:
            assert acc_gpu >= capacity
    filled = min(acc_ref, capacity)
    assert 0 < filled
    assert draw.ids.dtype == (torch.int64 if ids_int64 else torch.int32)
    np.testing.assert_array_equal(draw.ids.cpu().numpy()[:filled], ids_ref[:filled])
    np.testing.assert_array_equal(draw.pos.cpu().numpy()[:filled].view(np.uint32), pos_ref[:filled].view(np.uint32))
    draw.finish()
    rng_ref.advance(4 * (cons_ref if cons_ref else k0))
    assert H.rng_values(rng_dev) == (int(rng_ref.state[0]), int(rng_ref.state[1]))


def test_training_api_matches_oracle_draw(gpu, oracle):
    from inpc_amd import ProbabilityFieldSampler

    oct, hv = small_scene(distance=2.2)
    view = hv.to_view(gpu)
    sampler = ProbabilityFieldSampler(seed=9)
    rng_ref = oracle.Pcg32(9)
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    for n in (5000, 12345):  # two calls: the second continues the stream where the first stopped
        pos, ids = sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
        pos_ref, ids_ref, consumed = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c,
                                                             oracle_cam(oracle, hv), oct.initial_size, rng_ref, n)
        assert ids.dtype == torch.int64 and pos.shape == (n, 3)
        np.testing.assert_array_equal(ids.cpu().numpy(), ids_ref.astype(np.int64))
        np.testing.assert_array_equal(pos.cpu().numpy().view(np.uint32), pos_ref.view(np.uint32))
        assert sampler.last_consumed == consumed
        assert sampler.rng_state() == (int(rng_ref.state[0]), int(rng_ref.state[1]))


def test_training_api_draw_of_several_rounds(gpu, oracle):
    # A camera inside the octree: most candidates are rejected, the first round (sized for full acceptance) does not
    # complete the draw, and the end of the draw that was enqueued behind it must have changed nothing.
    from inpc_amd import ProbabilityFieldSampler

    oct, hv = small_scene(distance=0.6)
    view = hv.to_view(gpu)
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    sampler = ProbabilityFieldSampler(seed=21)
    rng_ref = oracle.Pcg32(21)
    n = 30000
    first_round = int(n * sampler.OVERSAMPLE) + 4096
    for _ in range(2):   # the second call starts from the acceptance the first one saw
        pos, ids = sampler.generate_training_samples(centers, levels, weights, view, n, oct.initial_size)
        pos_ref, ids_ref, consumed = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c,
                                                             oracle_cam(oracle, hv), oct.initial_size, rng_ref, n)
        np.testing.assert_array_equal(ids.cpu().numpy(), ids_ref.astype(np.int64))
        np.testing.assert_array_equal(pos.cpu().numpy().view(np.uint32), pos_ref.view(np.uint32))
        assert sampler.last_consumed == consumed
        assert sampler.rng_state() == (int(rng_ref.state[0]), int(rng_ref.state[1]))
    assert consumed > first_round, "the scene must need more than one round at full-acceptance sizing"


def test_training_api_failure_pattern(gpu):
    from inpc_amd import ProbabilityFieldSampler

    oct, hv = small_scene(300, 4)
    view = hv.to_view(gpu)
    sampler = ProbabilityFieldSampler(seed=1)
    before = sampler.rng_state()
    zero = torch.zeros(300, dtype=torch.float32, device=gpu)
    pos, ids = sampler.generate_training_samples(H.dev(oct.centers), H.dev(oct.levels), zero, view, 777,
                                                 oct.initial_size)
    assert (pos == 0).all() and (ids == -1).all()
    assert sampler.rng_state() == before
    empty = sampler.generate_samples(H.dev(oct.centers), H.dev(oct.levels), zero, view, 100, oct.initial_size)
    assert empty.shape == (0, 3)
    empty = sampler.generate_expected_samples(H.dev(oct.centers), H.dev(oct.levels), zero, view, 100, 2,
                                              oct.initial_size)
    assert empty.shape == (0, 3)


def test_generate_samples_and_expected_samples_api(gpu, oracle):
    from inpc_amd import ProbabilityFieldSampler, compute_viewpoint_weights

    oct, hv = small_scene()
    view = hv.to_view(gpu)
    cam = oracle_cam(oracle, hv)
    centers, levels, weights = H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights)
    w = compute_viewpoint_weights(centers, levels, weights, view, oct.initial_size)
    w_ref = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam, oct.initial_size)
    np.testing.assert_array_equal(w.cpu().numpy().view(np.uint32), w_ref.view(np.uint32))

    sampler = ProbabilityFieldSampler(seed=21)
    rng_ref = oracle.Pcg32(21)
    pos = sampler.generate_samples(centers, levels, weights, view, 33333, oct.initial_size)
    ok, cdf_ref, _ = oracle.build_cdf(w_ref)
    pos_ref, _ = oracle.sample(oct.centers, oct.levels, cdf_ref, 33333, oct.initial_size, rng_ref)
    np.testing.assert_array_equal(pos.cpu().numpy().view(np.uint32), pos_ref.view(np.uint32))

    out = sampler.generate_expected_samples(centers, levels, weights, view, 40000, 3, oct.initial_size)
    offs_ref, n_created, _ = oracle.expected_counts(w_ref, 40000)
    exp_ref = oracle.expected_samples(oct.centers, oct.levels, offs_ref, n_created, 3, oct.initial_size, rng_ref)
    assert out.shape == (n_created * 3, 3)
    np.testing.assert_array_equal(out.cpu().numpy().view(np.uint32), exp_ref.view(np.uint32))
    assert sampler.rng_state() == (int(rng_ref.state[0]), int(rng_ref.state[1]))


def test_expected_counts_without_a_positive_sum_are_all_zero(gpu):
    # no weight is positive (B/sampling/src/sampling_api.cu:196-199 returns no samples then): every offset is written
    # as zero whatever the buffers held before, the sum is reported, and the next call with weights works as usual
    lib = _lib.lib()
    n = 70001
    ws_bytes = lib.inpc_sampler_workspace_bytes(n)
    ws = H.poisoned_bytes(ws_bytes, gpu)
    offsets = torch.full((n,), 12345, dtype=torch.int32, device=gpu)
    total = torch.full((1,), 7.0, dtype=torch.float32, device=gpu)
    zeros = torch.zeros(n, dtype=torch.float32, device=gpu)
    _lib.check(lib.inpc_expected_counts(_lib.ptr(zeros), _lib.ptr(total), _lib.ptr(offsets), 1000, _lib.ptr(ws), ws_bytes,
                                        n, H.stream()), "inpc_expected_counts")
    assert float(total.item()) == 0.0
    assert int(offsets.abs().max().item()) == 0
    w = np.zeros(n, np.float32)
    w[[5, 4096, 70000]] = [1.0, 2.0, 1.0]
    w_dev = H.dev(w)   # kept alive over the call
    _lib.check(lib.inpc_expected_counts(_lib.ptr(w_dev), _lib.ptr(total), _lib.ptr(offsets), 1000, _lib.ptr(ws),
                                        ws_bytes, n, H.stream()), "inpc_expected_counts")
    assert float(total.item()) == 4.0
    got = offsets.cpu().numpy()
    want = np.zeros(n, np.int64)
    want[5:], want[4096:], want[70000:] = 250, 750, 1000
    np.testing.assert_array_equal(got, want)


def test_non_perspective_and_distorted_cameras_are_rejected(gpu):
    from inpc_amd import ProbabilityFieldSampler, compute_viewpoint_weights
    from inpc_amd.views import View

    oct, hv = small_scene(100, 4)
    view = hv.to_view(gpu)

    class Fisheye:
        width, height = 10, 10

    bad = View(Fisheye(), view.w2c, view.position)
    args = (H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights))
    with pytest.raises(NotImplementedError):
        compute_viewpoint_weights(*args, bad, 4.0)
    view.camera.distortion = object()
    with pytest.raises(NotImplementedError):
        ProbabilityFieldSampler(0).generate_samples(*args, view, 10, 4.0)


def test_training_draw_that_never_hits_the_frustum_is_filled_with_the_failure_pattern(gpu):
    # One leaf whose far face lies exactly on the near plane: its corners are visible, so its weight is positive, but
    # every jittered position inside it is nearer than the near plane and is culled. The draw gives up and the
    # samples it could not produce are position 0 / index -1, not whatever the buffers held.
    from inpc_amd import ProbabilityFieldSampler, synthetic

    hv = synthetic.camera_on_z(400, 300, 100.0, 0.0, near=1.0, far=50.0)   # camera at the origin, looking along +z
    centers = np.array([[0.0, 0.0, 0.5]], np.float32)                        # cube [-0.5, 0.5]^2 x [0, 1]
    levels = np.zeros(1, np.int32)
    weights = np.ones(1, np.float32)
    sampler = ProbabilityFieldSampler(seed=3)
    view = hv.to_view(gpu)
    w = H.leaf_weights(synthetic.Octree(centers, levels, weights, 1.0), hv)
    assert float(w[0].item()) > 0.0
    pos, ids = sampler.generate_training_samples(H.dev(centers), H.dev(levels), H.dev(weights), view, 1000, 1.0)
    assert pos.shape == (1000, 3) and ids.shape == (1000,)
    assert (pos == 0).all() and (ids == -1).all()
