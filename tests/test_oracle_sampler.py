"""Pins the oracle's sampler functions against closed forms, numpy routines and an independent PCG32 (CPU only)."""
import numpy as np
import pytest

from inpc_amd import synthetic
from tests.test_oracle_pcg32_and_half import PyPcg32


def cam_of(O, hv):
    c = hv.camera
    return O.make_camera(c.width, c.height, c.focal_x, c.focal_y, c.center_x, c.center_y, c.near_plane, c.far_plane)


def project64(hv, p):
    m = hv.w2c.astype(np.float64)
    q = p.astype(np.float64) @ m[:3, :3].T + m[:3, 3]
    c = hv.camera
    return q[:, 0] / q[:, 2] * c.focal_x + c.center_x, q[:, 1] / q[:, 2] * c.focal_y + c.center_y, q[:, 2]


def visible64(hv, p, margin=0.0):
    sx, sy, z = project64(hv, p)
    c = hv.camera
    return ((z >= c.near_plane + margin) & (z <= c.far_plane - margin) & (sx >= margin) & (sx < c.width - margin) &
            (sy >= margin) & (sy < c.height - margin))


def test_leaf_weights_closed_form(oracle):
    rng = np.random.default_rng(0)
    oct = synthetic.octree_leaves(5000, 6, 4.0, seed=1)
    oct.levels = rng.integers(2, 9, size=5000).astype(np.int32)
    hv = synthetic.rotated_camera(320, 200, 250.0, 3.0, 0.4, -0.2)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam_of(oracle, hv), oct.initial_size)
    # float64 restatement: visible if the centre or any corner projects inside the frustum
    half = oct.initial_size / 2.0 ** (oct.levels + 1)
    vis = visible64(hv, oct.centers)
    for corner in range(8):
        off = np.array([(corner >> 2) & 1, (corner >> 1) & 1, corner & 1]) * 2.0 - 1.0
        vis |= visible64(hv, oct.centers + half[:, None] * off)
    _, _, z = project64(hv, oct.centers)
    c = hv.camera
    expect = oct.weights / (np.maximum(np.abs(z - c.near_plane) / c.far_plane, 1e-8) * 2.0 ** (oct.levels / 2.0))
    expect = np.where(vis, expect, 0.0)
    # leaves whose visibility hinges on rounding at the frustum border are excluded
    border = np.zeros(5000, bool)
    for corner in range(-1, 8):
        off = np.zeros(3) if corner < 0 else np.array([(corner >> 2) & 1, (corner >> 1) & 1, corner & 1]) * 2.0 - 1.0
        p = oct.centers + half[:, None] * off
        border |= visible64(hv, p, -1e-3) != visible64(hv, p, 1e-3)
    keep = ~border
    assert keep.mean() > 0.9 and (expect[keep] > 0).sum() > 500 and (expect[keep] == 0).sum() > 50
    np.testing.assert_allclose(w[keep], expect[keep], rtol=2e-6, atol=0)


def test_leaf_weight_constructed_cases(oracle):
    hv = synthetic.camera_on_z(100, 100, 100.0, 5.0)  # sees |x|,|y| < z/2 around the axis
    cam = cam_of(oracle, hv)
    centers = np.array([[0, 0, 0],          # centre visible
                        [2.9, 0, 0],        # centre outside (x limit at z=5 is 2.5), a corner inside
                        [30, 0, 0],         # nothing visible
                        [0, 0, -20]],       # behind the camera
                       dtype=np.float32)
    levels = np.array([3, 1, 3, 3], np.int32)   # level 1 of size 4: half edge 1.0
    w = oracle.leaf_weights(centers, levels, np.ones(4, np.float32), hv.w2c, cam, 4.0)
    assert w[0] > 0 and w[1] > 0 and w[2] == 0 and w[3] == 0
    # weight falls with depth and with level (w / (depth_scale * 2^(level/2)))
    c2 = np.array([[0, 0, 0], [0, 0, 2], [0, 0, 0]], np.float32)
    w2 = oracle.leaf_weights(c2, np.array([3, 3, 5], np.int32), np.ones(3, np.float32), hv.w2c, cam, 4.0)
    assert w2[0] > w2[1] and w2[0] == pytest.approx(2.0 * w2[2], rel=1e-6)
    assert w2[0] == pytest.approx(1.0 / ((5.0 - 0.01) / 100.0 * 2.0 ** 1.5), rel=1e-6)


@pytest.mark.parametrize("n", [1, 5, 63, 64, 65, 4095, 4096, 4097, 70001, 300000])
def test_blocked_scan_exact_on_integers(oracle, n):
    # small integers add exactly in fp32 whatever the association: pins indexing against numpy's cumsum
    rng = np.random.default_rng(n)
    w = rng.integers(0, 16, size=n).astype(np.float32)
    np.testing.assert_array_equal(oracle.blocked_inclusive_scan(w), np.cumsum(w.astype(np.int64)).astype(np.float32))
    assert float(oracle.blocked_total(w)) == float(w.astype(np.int64).sum())


def test_blocked_scan_close_to_float64_and_monotone(oracle):
    rng = np.random.default_rng(3)
    w = np.exp(rng.normal(0, 1.5, size=262144)).astype(np.float32)
    w[rng.random(262144) < 0.3] = 0.0
    ok, cdf, total = oracle.build_cdf(w)
    assert ok
    ref = np.cumsum(w.astype(np.float64))
    assert float(total) == pytest.approx(ref[-1], rel=1e-6)
    np.testing.assert_allclose(cdf, ref / ref[-1], rtol=0, atol=2e-6)
    assert abs(float(cdf[-1]) - 1.0) < 1e-5
    chunks = cdf[: (len(cdf) // 64) * 64].reshape(-1, 64)
    assert (np.diff(chunks, axis=1) >= 0).all()  # left-to-right sums of non-negative terms never decrease


def test_build_cdf_failure_leaves_input(oracle):
    w = np.zeros(1000, np.float32)
    ok, cdf, total = oracle.build_cdf(w)
    assert not ok and float(total) == 0.0
    np.testing.assert_array_equal(cdf, w)


def test_cdf_search_is_lower_bound(oracle):
    rng = np.random.default_rng(5)
    cdf = np.cumsum(rng.random(1000)).astype(np.float32)
    cdf /= cdf[-1]
    cdf[100:110] = cdf[100]  # plateaus (zero-weight leaves)
    samples = np.concatenate([rng.random(2000).astype(np.float32), cdf[::37], [0.0, 1.0, 2.0]]).astype(np.float32)
    expect = np.minimum(np.searchsorted(cdf, samples, side="left"), len(cdf) - 1)
    got = np.array([oracle.cdf_search(cdf, float(u)) for u in samples])
    np.testing.assert_array_equal(got, expect)


def small_tree(seed=2):
    oct = synthetic.octree_leaves(3000, 6, 4.0, seed=seed)
    oct.levels = np.random.default_rng(seed).integers(3, 8, size=3000).astype(np.int32)
    return oct


def test_sample_matches_independent_draws(oracle):
    # candidate k uses the generator advanced by 4k: u, then the three jitters
    oct = small_tree()
    hv = synthetic.camera_on_z(200, 150, 180.0, 3.5)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam_of(oracle, hv), oct.initial_size)
    ok, cdf, _ = oracle.build_cdf(w)
    n = 500
    rng = oracle.Pcg32(321)
    before = rng.copy()
    pos, ids = oracle.sample(oct.centers, oct.levels, cdf, n, oct.initial_size, rng)
    py = PyPcg32(321, 1)
    for k in range(n):
        u, ox, oy, oz = (py.next_float() for _ in range(4))
        leaf = min(int(np.searchsorted(cdf, u, side="left")), len(cdf) - 1)
        assert ids[k] == leaf
        scale = np.float32(np.float32(2.0 ** -int(oct.levels[leaf])) * np.float32(oct.initial_size))
        expect = oct.centers[leaf] + (np.array([ox, oy, oz], np.float32) - np.float32(0.5)) * scale
        assert pos[k].tobytes() == expect.astype(np.float32).tobytes()
    before.advance(4 * n)
    assert int(rng.state[0]) == int(before.state[0])  # the stream continues behind the draw


def test_sample_statistics_and_bounds(oracle):
    oct = small_tree(4)
    hv = synthetic.camera_on_z(200, 150, 180.0, 3.5)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam_of(oracle, hv), oct.initial_size)
    ok, cdf, total = oracle.build_cdf(w)
    n = 400000
    pos, ids = oracle.sample(oct.centers, oct.levels, cdf, n, oct.initial_size, oracle.Pcg32(1))
    size = oct.initial_size / 2.0 ** oct.levels[ids]
    assert (np.abs(pos - oct.centers[ids]) <= size[:, None] / 2 + 1e-6).all()
    assert (w[ids] > 0).all()  # zero-weight leaves are never picked
    p = w.astype(np.float64) / w.astype(np.float64).sum()
    counts = np.bincount(ids, minlength=len(w))
    sel = p * n > 20
    chi2 = (((counts[sel] - p[sel] * n) ** 2) / (p[sel] * n)).sum()
    dof = sel.sum()
    assert abs(chi2 - dof) < 6 * np.sqrt(2 * dof)


def accepted32(hv, p):
    """The rejection test of the training sampler, in fp32 in the reference's evaluation order."""
    m = hv.w2c.astype(np.float32)
    c = hv.camera
    f32 = np.float32
    row = lambda r: ((m[r, 0] * p[:, 0] + m[r, 1] * p[:, 1]) + m[r, 2] * p[:, 2]) + m[r, 3]
    z = row(2)
    inv = f32(1.0) / (z + f32(1e-8))
    sx = row(0) * inv * f32(c.focal_x) + f32(c.center_x)
    sy = row(1) * inv * f32(c.focal_y) + f32(c.center_y)
    return ~((z < f32(c.near_plane)) | (z > f32(c.far_plane)) | (sx < 0) | (sx >= f32(c.width)) | (sy < 0) |
             (sy >= f32(c.height)))


def test_cull_compact_is_the_filtered_candidate_stream(oracle):
    oct = small_tree(6)
    hv = synthetic.camera_on_z(200, 150, 180.0, 2.2)  # close: many candidates fall outside
    cam = cam_of(oracle, hv)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam, oct.initial_size)
    ok, cdf, _ = oracle.build_cdf(w)
    m = 60000
    cand_pos, cand_ids = oracle.sample(oct.centers, oct.levels, cdf, m, oct.initial_size, oracle.Pcg32(11))
    keep = accepted32(hv, cand_pos)
    assert 0.2 < keep.mean() < 0.98
    capacity = int(keep.sum()) - 100
    # one round, and the same draw cut into ragged rounds
    for rounds in ([m], [1, 4095, 4096, 4097, m - 12289]):
        pos = ids = None
        accepted, consumed, k0 = 0, 0, 0
        rng = oracle.Pcg32(11)
        for r in rounds:
            pos, ids, accepted, c = oracle.sample_cull_compact(oct.centers, oct.levels, cdf, hv.w2c, cam,
                                                               oct.initial_size, rng, capacity, k0, r, pos, ids,
                                                               accepted)
            consumed = c or consumed
            k0 += r
        assert accepted == keep.sum()
        np.testing.assert_array_equal(ids, cand_ids[keep][:capacity])
        np.testing.assert_array_equal(pos.view(np.uint32), cand_pos[keep][:capacity].view(np.uint32))
        assert consumed == np.flatnonzero(keep)[capacity - 1] + 1
    assert visible64(hv, pos, -1e-3).all()  # every emitted point is inside the frustum


def test_training_draw_advances_by_consumed_candidates(oracle):
    oct = small_tree(7)
    hv = synthetic.camera_on_z(200, 150, 180.0, 2.2)
    cam = cam_of(oracle, hv)
    rng = oracle.Pcg32(3)
    start = rng.copy()
    n = 20000
    pos, ids, consumed = oracle.training_samples(oct.centers, oct.levels, oct.weights, hv.w2c, cam, oct.initial_size,
                                                 rng, n)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam, oct.initial_size)
    ok, cdf, _ = oracle.build_cdf(w)
    cand_pos, cand_ids = oracle.sample(oct.centers, oct.levels, cdf, consumed, oct.initial_size, start.copy())
    keep = accepted32(hv, cand_pos)
    assert keep.sum() == n and keep[-1]  # exactly n accepted, the last consumed candidate is the n-th
    np.testing.assert_array_equal(ids, cand_ids[keep])
    start.advance(4 * consumed)
    assert int(rng.state[0]) == int(start.state[0])
    # failure path: nothing visible
    zero = np.zeros_like(oct.weights)
    rng2 = oracle.Pcg32(3)
    pos, ids, consumed = oracle.training_samples(oct.centers, oct.levels, zero, hv.w2c, cam, oct.initial_size, rng2, 50)
    assert (pos == 0).all() and (ids == -1).all() and consumed == 0
    assert int(rng2.state[0]) == int(oracle.Pcg32(3).state[0])


def test_expected_counts_and_samples(oracle):
    oct = small_tree(8)
    hv = synthetic.camera_on_z(200, 150, 180.0, 3.5)
    w = oracle.leaf_weights(oct.centers, oct.levels, oct.weights, hv.w2c, cam_of(oracle, hv), oct.initial_size)
    n = 50000
    offs, n_created, total = oracle.expected_counts(w, n)
    norm = np.float32(1.0) / np.float32(total)
    expect = np.where(w > 0, np.maximum(np.rint((w * norm) * np.float32(n)), 1), 0).astype(np.int64)  # half to even
    np.testing.assert_array_equal(np.diff(np.concatenate([[0], offs])), expect)
    assert n_created == expect.sum()
    rng = oracle.Pcg32(5)
    start = rng.copy()
    pos = oracle.expected_samples(oct.centers, oct.levels, offs, n_created, 2, oct.initial_size, rng)
    ids = np.repeat(np.arange(len(w)), expect)
    leaf = np.concatenate([ids, ids])  # sample j lies in leaf ids[j mod n_created]
    size = oct.initial_size / 2.0 ** oct.levels[leaf]
    assert (np.abs(pos - oct.centers[leaf]) <= size[:, None] / 2 + 1e-6).all()
    py = PyPcg32(5, 1)
    for j in range(3):  # sample j uses the generator advanced by 3j
        o = np.array([py.next_float() for _ in range(3)], np.float32)
        scale = np.float32(np.float32(2.0 ** -int(oct.levels[leaf[j]])) * np.float32(oct.initial_size))
        assert pos[j].tobytes() == (oct.centers[leaf[j]] + (o - np.float32(0.5)) * scale).astype(np.float32).tobytes()
    start.advance(3 * 2 * n_created)
    assert int(rng.state[0]) == int(start.state[0])
    assert oracle.expected_counts(np.zeros(10, np.float32), 100)[1] == 0
