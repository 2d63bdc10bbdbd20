"""Pins the oracle's probability-field update against the reference's own formulation (the torch calls of
Modules/ProbabilityField.py:146-157, evaluated by torch on the CPU) and against hand-checked cases."""
import numpy as np
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
