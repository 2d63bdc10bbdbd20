"""Pins the oracle's probability-field update against the reference's own formulation (the torch calls of
Modules/ProbabilityField.py:146-157, evaluated by torch on the CPU) and against hand-checked cases."""
import numpy as np
import pytest
import torch


def reference_formulation(leaf_weights, leaf_scores, indices, weights):
    lw = torch.tensor(leaf_weights).clone()
    ls = torch.tensor(leaf_scores).clone()
    idx = torch.tensor(indices)
    lw.mul_(0.9968)
    ls.mul_(0.9968)
    w = torch.tensor(weights).squeeze().to(lw)
    max_sampled = torch.zeros_like(lw)
    min_sampled = torch.zeros_like(lw)
    max_sampled.scatter_reduce_(dim=0, index=idx, src=w, reduce='amax', include_self=False)
    min_sampled.scatter_reduce_(dim=0, index=idx, src=w, reduce='amin', include_self=False)
    torch.maximum(lw, max_sampled, out=lw)
    torch.maximum(ls, max_sampled.sub_(min_sampled).clamp_(0.0, 1.0), out=ls)
    return lw.numpy(), ls.numpy()


def test_matches_the_torch_formulation_bit_for_bit(oracle):
    rng = np.random.default_rng(0)
    for n_leaves, n_samples in [(1, 5), (100, 0), (1000, 300), (5000, 200000)]:
        lw = rng.random(n_leaves).astype(np.float32)
        ls = rng.random(n_leaves).astype(np.float32)
        idx = rng.integers(0, n_leaves, n_samples).astype(np.int64)
        w = (rng.random((n_samples, 1)) ** 3).astype(np.float32) * 1.5   # some weights above 1: the clamp acts
        a, b = oracle.field_update(lw, ls, idx, w)
        ra, rb = reference_formulation(lw, ls, idx, w)
        np.testing.assert_array_equal(a.view(np.uint32), ra.view(np.uint32))
        np.testing.assert_array_equal(b.view(np.uint32), rb.view(np.uint32))


def test_hand_checked_case(oracle):
    lw = np.array([0.5, 0.5, 0.0, 1.0], np.float32)
    ls = np.array([0.0, 0.9, 0.0, 0.0], np.float32)
    idx = np.array([0, 0, 0, 1, 3], np.int64)
    w = np.array([0.2, 0.9, 0.4, 0.1, 3.0], np.float32)
    a, b = oracle.field_update(lw, ls, idx, w)
    d = np.float32(0.9968)
    np.testing.assert_array_equal(a, np.array([0.9, np.float32(0.5) * d, 0.0, 3.0], np.float32))
    # leaf 0: spread 0.9 - 0.2; leaf 1: one sample -> spread 0, the decayed score stays; leaf 2: no sample; leaf 3: one sample
    np.testing.assert_array_equal(b, np.array([np.float32(0.9) - np.float32(0.2), np.float32(0.9) * d, 0.0, 0.0], np.float32))


def test_order_of_the_samples_does_not_matter(oracle):
    rng = np.random.default_rng(1)
    lw, ls = rng.random(300).astype(np.float32), rng.random(300).astype(np.float32)
    idx = rng.integers(0, 300, 5000).astype(np.int64)
    w = rng.random(5000).astype(np.float32)
    p = rng.permutation(5000)
    a, b = oracle.field_update(lw, ls, idx, w)
    a2, b2 = oracle.field_update(lw, ls, idx[p], w[p])
    np.testing.assert_array_equal(a, a2)
    np.testing.assert_array_equal(b, b2)


def _random_octree(rng, n):
    centers = rng.uniform(-2, 2, (n, 3)).astype(np.float32)
    levels = rng.integers(0, 8, n).astype(np.int32)
    weights = rng.random(n).astype(np.float32)
    scores = rng.random(n).astype(np.float32)
    return centers, levels, weights, scores


def test_prune_matches_the_references_torch_statements(oracle):
    # Modules/ProbabilityField.py:159-165 run by torch on the CPU
    rng = np.random.default_rng(21)
    centers, levels, weights, scores = _random_octree(rng, 5000)
    weights[::7] = 0.25  # values on the threshold are dropped (strict comparison)
    mask = torch.from_numpy(weights) > 0.25
    want = [torch.from_numpy(a)[mask].contiguous().numpy() for a in (centers, levels, weights, scores)]
    got = oracle.field_prune(centers, levels, weights, scores, 0.25)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g, w)
    assert len(got[0]) < 5000 and (got[2] > 0.25).all()


def test_subdivide_matches_the_references_torch_statements(oracle):
    # Modules/ProbabilityField.py:217-257 run by torch on the CPU, statement by statement
    rng = np.random.default_rng(22)
    centers, levels, weights, scores = _random_octree(rng, 3000)
    initial = torch.tensor([0.37, 0.37, 0.37], dtype=torch.float32)
    threshold = 0.6
    c, l, w, s = (torch.from_numpy(a) for a in (centers, levels, weights, scores))
    valid_mask = (s > threshold) & (l < 6)
    valid_centers, valid_levels, valid_weights = c[valid_mask], l[valid_mask], w[valid_mask]
    new_centers = torch.repeat_interleave(valid_centers, 8, dim=0)
    new_levels = torch.repeat_interleave(valid_levels + 1, 8, dim=0)
    new_weights = torch.repeat_interleave(valid_weights, 8, dim=0)
    new_scores = torch.zeros_like(new_weights)
    offset = initial / (2 ** (new_levels + 1))[:, None]
    new_centers[0::2, 0] -= offset[0::2, 0]
    new_centers[1::2, 0] += offset[1::2, 0]
    new_centers[0::4, 1] -= offset[0::4, 1]
    new_centers[1::4, 1] -= offset[1::4, 1]
    new_centers[2::4, 1] += offset[2::4, 1]
    new_centers[3::4, 1] += offset[3::4, 1]
    for k in range(4):
        new_centers[k::8, 2] -= offset[k::8, 2]
        new_centers[4 + k::8, 2] += offset[4 + k::8, 2]
    want = (torch.cat([c[~valid_mask], new_centers]), torch.cat([l[~valid_mask], new_levels]),
            torch.cat([w[~valid_mask], new_weights]), torch.cat([s[~valid_mask], new_scores]))
    got = oracle.field_subdivide(centers, levels, weights, scores, initial.numpy(), threshold)
    assert int(valid_mask.sum()) > 100 and (levels[valid_mask.numpy()] < 6).all()
    for g, t in zip(got, want):
        np.testing.assert_array_equal(g, t.numpy())
    # the size limit of :223-224
    assert oracle.field_subdivide(centers, levels, weights, scores, initial.numpy(), threshold, max_leaves=3500) is None


def _reference_halton_base(index, base):
    # utils.py:36-45
    result = 0
    f = 1 / base
    i = index
    while i > 0:
        result += f * (i % base)
        i = i // base
        f /= base
    return result


def test_extract_global_matches_the_references_torch_statements(oracle):
    # Modules/ProbabilityField.py:131-140 and utils.py:48-64 run by torch on the CPU, statement by statement
    rng = np.random.default_rng(23)
    n_leaves = 400
    centers = torch.from_numpy(rng.uniform(-2, 2, (n_leaves, 3)).astype(np.float32))
    levels = torch.from_numpy(rng.integers(0, 7, n_leaves).astype(np.int32))
    initial = torch.tensor([0.37, 0.37, 0.37], dtype=torch.float32)
    indices = torch.from_numpy(rng.integers(0, n_leaves, 900))
    indices[:40] = 7           # one crowded leaf, many leaves with a single sample or none
    counts = torch.bincount(indices, minlength=n_leaves)
    cell = torch.arange(n_leaves, dtype=torch.int32).repeat_interleave(counts)
    offsets = torch.cumsum(counts, dim=0) - counts
    halton_indices = torch.arange(counts.sum().item(), dtype=torch.int32) - offsets[cell]
    table = torch.zeros((halton_indices.max().item() + 1, 3))
    for i in range(table.shape[0]):
        for j, prime in enumerate([2, 3, 5]):
            table[i][j] = _reference_halton_base(i + 1, prime)
    halton_coords = table[halton_indices]
    cell_size = initial / 2 ** levels[cell, None]
    initial_samples = centers[cell]
    samples = initial_samples - (cell_size / 2) + halton_coords * cell_size
    single = (counts == 1).repeat_interleave(counts)
    samples[single] = initial_samples[single]
    got = oracle.extract_global_samples(centers.numpy(), levels.numpy(), initial.numpy(), counts.numpy())
    assert (counts == 1).sum() > 5 and (counts == 0).sum() > 0 and counts.max() >= 40
    np.testing.assert_array_equal(got.view(np.uint32), samples.numpy().view(np.uint32))
    # the first Halton points, as published: 1/2, 1/3, 1/5; 1/4, 2/3, 2/5; 3/4, 1/9, 3/5
    assert [oracle.halton_base(1, b) for b in (2, 3, 5)] == pytest.approx([1 / 2, 1 / 3, 1 / 5])
    assert [oracle.halton_base(3, b) for b in (2, 3, 5)] == pytest.approx([3 / 4, 1 / 9, 3 / 5])


def test_morton_codes_are_the_z_order_of_the_bounding_cube(oracle):
    # a lattice whose bounding cube is [0, 2^21]^3: the scale is exactly 1 and a cell is the coordinate itself
    top = float(2 ** 21)
    lattice = np.array([[0, 0, 0], [1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1], [2, 0, 0], [3, 5, 6],
                        [2 ** 21 - 1, 0, 0], [0, 2 ** 21 - 1, 2 ** 21 - 1], [top, top, top]], np.float32)
    codes = oracle.morton_encode(lattice)
    x_bits = sum(1 << (3 * k) for k in range(21))
    assert codes.tolist() == [0, 1, 2, 4, 7, 8, 0b110_101_011, x_bits, 6 * x_bits, 7 * x_bits]   # the corner is clamped
    assert codes.dtype == np.int64 and (codes >= 0).all()
    # a 4 x 4 x 4 lattice sorted by code: octant by octant, x fastest inside each 2 x 2 x 2 block
    g = np.stack(np.meshgrid(np.arange(4), np.arange(4), np.arange(4), indexing="ij"), -1).reshape(-1, 3)
    pts = np.concatenate([g.astype(np.float32) * np.float32(2 ** 19), [[top, top, top]]]).astype(np.float32)
    order = np.argsort(oracle.morton_encode(pts)[:-1], kind="stable")
    walk = g[order]
    first_block = [[0, 0, 0], [1, 0, 0], [0, 1, 0], [1, 1, 0], [0, 0, 1], [1, 0, 1], [0, 1, 1], [1, 1, 1]]
    assert walk[:8].tolist() == first_block
    assert (walk[8:16] - [2, 0, 0]).tolist() == first_block and (walk[16:24] - [0, 2, 0]).tolist() == first_block
    assert (walk[56:] - [2, 2, 2]).tolist() == first_block
    # a shift and a scaling by powers of two change no cell (every float operation stays exact)
    rng = np.random.default_rng(31)
    p = rng.integers(0, 2 ** 21, (5000, 3)).astype(np.float32)
    p[0], p[1] = 0.0, top
    np.testing.assert_array_equal(oracle.morton_encode(p * np.float32(0.25) - np.float32(1024.0)), oracle.morton_encode(p))
    # the largest extent sets the cube: the short axes only use the lower cells
    q = p * np.array([1.0, 0.5, 0.25], np.float32)
    cells_y = sum(((oracle.morton_encode(q) >> (3 * k + 1)) & 1) << k for k in range(21))
    assert cells_y.max() < 2 ** 20 + 1
    # one point, identical points, no points
    assert oracle.morton_encode(np.array([[1.5, -2.0, 3.0]], np.float32)).tolist() == [0]
    assert oracle.morton_encode(np.full((7, 3), 0.25, np.float32)).tolist() == [0] * 7
    assert oracle.morton_encode(np.zeros((0, 3), np.float32)).shape == (0,)
