"""GPU parity of the probability-field update against the oracle, through the C ABI and the Python operator.
Maximum and minimum are order independent: every output is bit-exact."""
import numpy as np
import pytest
import torch

from inpc_amd import _lib, update_probability_field
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_leaves,n_samples", [(1, 7), (63, 0), (1000, 257), (262144, 1 << 20)])
def test_update_bit_exact(gpu, oracle, n_leaves, n_samples):
    rng = np.random.default_rng(n_leaves)
    lw = rng.random(n_leaves).astype(np.float32)
    ls = rng.random(n_leaves).astype(np.float32)
    idx = rng.integers(0, n_leaves, n_samples).astype(np.int64)
    w = (rng.random(n_samples) ** 3 * 1.5).astype(np.float32)
    w[::97] = -0.25 * w[::97]                      # signs are handled too
    d_lw, d_ls, d_idx, d_w = H.dev(lw), H.dev(ls), H.dev(idx), H.dev(w.reshape(-1, 1))
    update_probability_field(d_lw, d_ls, d_idx, d_w, check=True)
    a, b = oracle.field_update(lw, ls, idx, w)
    np.testing.assert_array_equal(d_lw.cpu().numpy().view(np.uint32), a.view(np.uint32))
    np.testing.assert_array_equal(d_ls.cpu().numpy().view(np.uint32), b.view(np.uint32))


def test_two_updates_in_a_row_and_bad_index(gpu, oracle):
    rng = np.random.default_rng(5)
    lw = rng.random(500).astype(np.float32)
    ls = np.zeros(500, np.float32)
    d_lw, d_ls = H.dev(lw), H.dev(ls)
    for step in range(2):
        idx = rng.integers(0, 500, 3000).astype(np.int64)
        w = rng.random(3000).astype(np.float32)
        update_probability_field(d_lw, d_ls, H.dev(idx), H.dev(w))
        lw, ls = oracle.field_update(lw, ls, idx, w)
    np.testing.assert_array_equal(d_lw.cpu().numpy(), lw)
    np.testing.assert_array_equal(d_ls.cpu().numpy(), ls)
    bad = np.array([0, 500, 3], np.int64)
    with pytest.raises(_lib.BackendError, match="outside"):
        update_probability_field(d_lw, d_ls, H.dev(bad), H.dev(np.ones(3, np.float32)), check=True)


def test_closes_the_loop_with_sampler_and_rasterizer(gpu, oracle):
    """indices from generate_training_samples + blending weights from the rasterizer -> field update."""
    from inpc_amd import ProbabilityFieldSampler, synthetic
    from inpc_amd.rasterization import rasterize_points

    oct = synthetic.octree_leaves(4096, 5, 4.0, seed=3)
    hv = synthetic.camera_on_z(160, 120, 140.0, 6.0)
    view = hv.to_view(gpu)
    sampler = ProbabilityFieldSampler(seed=1)
    pos, ids = sampler.generate_training_samples(H.dev(oct.centers), H.dev(oct.levels), H.dev(oct.weights), view, 50000,
                                                 oct.initial_size)
    gen = torch.Generator(device=gpu).manual_seed(2)
    feats = torch.randn((50000, 4), generator=gen, device=gpu)
    opac = torch.sigmoid(torch.randn(50000, generator=gen, device=gpu))
    _, _, bw = rasterize_points(view, pos, feats, opac, tile=16)
    lw = np.full(4096, 0.01, np.float32)
    ls = np.zeros(4096, np.float32)
    d_lw, d_ls = H.dev(lw), H.dev(ls)
    update_probability_field(d_lw, d_ls, ids, bw, check=True)
    a, b = oracle.field_update(lw, ls, ids.cpu().numpy(), bw.cpu().numpy())
    np.testing.assert_array_equal(d_lw.cpu().numpy(), a)
    np.testing.assert_array_equal(d_ls.cpu().numpy(), b)
    assert (a > np.float32(0.01) * np.float32(0.9968)).sum() > 100   # sampled leaves took their maxima


def _octree(rng, n):
    centers = rng.uniform(-2, 2, (n, 3)).astype(np.float32)
    levels = rng.integers(0, 8, n).astype(np.int32)
    return centers, levels, rng.random(n).astype(np.float32), rng.random(n).astype(np.float32)


@pytest.mark.parametrize("n", [1, 1023, 1024, 70001])
def test_prune_bit_exact(gpu, oracle, n):
    from inpc_amd import prune_probability_field

    rng = np.random.default_rng(n)
    arrays = _octree(rng, n)
    got = prune_probability_field(*(H.dev(a) for a in arrays), 0.4)
    want = oracle.field_prune(*arrays, 0.4)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)


def test_prune_everything_and_nothing(gpu, oracle):
    from inpc_amd import prune_probability_field

    arrays = _octree(np.random.default_rng(5), 3000)
    assert all(t.shape[0] == 0 for t in prune_probability_field(*(H.dev(a) for a in arrays), 2.0))
    kept = prune_probability_field(*(H.dev(a) for a in arrays), -1.0)
    for g, a in zip(kept, arrays):
        np.testing.assert_array_equal(g.cpu().numpy(), a)


@pytest.mark.parametrize("n", [1, 1024, 33333])
def test_subdivide_bit_exact(gpu, oracle, n):
    from inpc_amd import subdivide_probability_field

    rng = np.random.default_rng(100 + n)
    arrays = _octree(rng, n)
    size = np.array([0.37, 0.37, 0.37], np.float32)
    got = subdivide_probability_field(*(H.dev(a) for a in arrays), torch.from_numpy(size), 0.55)
    want = oracle.field_subdivide(*arrays, size, 0.55)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)
    # the size limit: nothing is returned, as the reference leaves the octree alone
    n_split = (len(want[1]) - n) // 7
    if n_split:
        assert subdivide_probability_field(*(H.dev(a) for a in arrays), size, 0.55, max_leaves=len(want[1]) - 1) is None


def test_extract_global_bit_exact(gpu, oracle):
    from inpc_amd import extract_global_samples

    rng = np.random.default_rng(9)
    n_leaves = 5000
    centers = rng.uniform(-2, 2, (n_leaves, 3)).astype(np.float32)
    levels = rng.integers(0, 7, n_leaves).astype(np.int32)
    size = np.array([0.37, 0.37, 0.37], np.float32)
    indices = rng.integers(0, n_leaves, 40000)
    indices[:3000] = 11         # one crowded leaf
    indices = indices[indices % 5 != 0]   # a fifth of the leaves stays empty
    counts = np.bincount(indices, minlength=n_leaves).astype(np.int64)
    got = extract_global_samples(H.dev(centers), H.dev(levels), size, H.dev(counts)).cpu().numpy()
    want = oracle.extract_global_samples(centers, levels, size, counts)
    assert (counts == 1).sum() > 10 and (counts == 0).sum() > 100
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    # inside the cell
    cell = np.repeat(np.arange(n_leaves), counts)
    half = (size[None, :] / (2.0 ** levels[cell])[:, None]) / 2
    assert (np.abs(got - centers[cell]) <= half * (1 + 1e-6)).all()
    with pytest.raises(RuntimeError):
        bad = counts.copy()
        bad[0] = -1
        extract_global_samples(H.dev(centers), H.dev(levels), size, H.dev(bad))


def test_morton_codes_bit_exact_and_the_ordered_extraction(gpu, oracle):
    from inpc_amd import extract_global_samples, morton_encode

    rng = np.random.default_rng(41)
    for n, spread in ((1, 1.0), (2, 1.0), (63, 1e-3), (200001, 3.0)):
        p = (rng.normal(0, spread, (n, 3)) * np.array([1.0, 0.3, 2.0])).astype(np.float32)
        got = morton_encode(H.dev(p)).cpu().numpy()
        np.testing.assert_array_equal(got, oracle.morton_encode(p), err_msg=f"n = {n}")
    assert morton_encode(H.dev(np.full((100, 3), -0.75, np.float32))).cpu().numpy().tolist() == [0] * 100
    assert morton_encode(H.dev(np.zeros((0, 3), np.float32))).shape == (0,)
    with pytest.raises(RuntimeError):
        morton_encode(H.dev(np.zeros((4, 2), np.float32)))
    # extract_global with use_morton_order: the same samples, in the order of their codes
    n_leaves = 3000
    centers = rng.uniform(-2, 2, (n_leaves, 3)).astype(np.float32)
    levels = rng.integers(0, 7, n_leaves).astype(np.int32)
    size = np.array([0.37, 0.37, 0.37], np.float32)
    counts = np.bincount(rng.integers(0, n_leaves, 20000), minlength=n_leaves).astype(np.int64)
    plain = oracle.extract_global_samples(centers, levels, size, counts)
    got = extract_global_samples(H.dev(centers), H.dev(levels), size, H.dev(counts), use_morton_order=True).cpu().numpy()
    codes = oracle.morton_encode(plain)
    np.testing.assert_array_equal(oracle.morton_encode(got), np.sort(codes))   # the same cube, so the same codes
    rows = lambda a: a[np.lexsort(a.T[::-1])]
    np.testing.assert_array_equal(rows(got).view(np.uint32), rows(plain).view(np.uint32))
