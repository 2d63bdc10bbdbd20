"""Pins the oracle's element-wise operators: closed forms in float64, the properties the contraction is used for,
and torch autograd through the reference's own expression for the opacity gradient."""
import numpy as np
import torch


def test_spherical_contraction_closed_form_and_properties(oracle):
    rng = np.random.default_rng(0)
    p = (rng.normal(size=(20000, 3)) * rng.choice([0.2, 1.0, 5.0, 100.0], size=(20000, 1))).astype(np.float32)
    out = oracle.spherical_contraction(p)
    p64 = p.astype(np.float64)
    r = np.linalg.norm(p64, axis=1, keepdims=True)
    inside = r <= 1
    # the usual contraction: p inside the unit ball, (2 - 1/|p|) p/|p| outside, then mapped from [-2,2] to [0,1]
    contracted = np.where(inside, p64, (2 - 1 / np.maximum(r, 1e-30)) * p64 / np.maximum(r, 1e-30))
    np.testing.assert_allclose(out, np.clip(contracted / 4 + 0.5, 0, 1), rtol=0, atol=2e-7)
    assert out.min() >= 0 and out.max() <= 1
    # inside the unit ball the map is p / 4 + 0.5 exactly as written (scale = 0.25)
    small = p[inside[:, 0]]
    np.testing.assert_array_equal(oracle.spherical_contraction(small), (np.float32(0.25) * small + np.float32(0.5)))
    # far points approach the boundary of the ball of radius 1/2 around the centre of the cube
    far = oracle.spherical_contraction(np.array([[1e6, 0, 0], [0, -1e6, 0]], np.float32))
    np.testing.assert_allclose(far, [[1.0, 0.5, 0.5], [0.5, 0.0, 0.5]], atol=1e-6)


def test_opacity_against_float64_and_autograd(oracle):
    x = np.linspace(-20, 6, 4001).astype(np.float32)
    out = oracle.feature_to_opacity(x)
    np.testing.assert_allclose(out, -np.expm1(-np.exp(x.astype(np.float64))), rtol=2e-6, atol=1e-12)
    assert (out >= 0).all() and (out <= 1).all() and (np.diff(out) >= 0).all()
    # gradient: torch autograd through -expm1(-exp(x)) in float64; inside [-15, 15] the truncation does not act
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    g = np.random.default_rng(1).normal(size=x.shape).astype(np.float32)
    (-torch.expm1(-torch.exp(xt))).backward(torch.tensor(g.astype(np.float64)))
    ours = oracle.feature_to_opacity_backward(g, x)
    sel = np.abs(x) <= 15
    np.testing.assert_allclose(ours[sel], xt.grad.numpy()[sel], rtol=5e-6, atol=1e-12)
    # outside, the inner exponential's gradient is frozen at exp(+-15)
    big = np.array([-18.0, -16.0], np.float32)
    expect = np.exp(-np.exp(big.astype(np.float64))) * np.exp(-15.0)
    np.testing.assert_allclose(oracle.feature_to_opacity_backward(np.ones(2, np.float32), big), expect, rtol=5e-6)


def test_weight_decay_factors(oracle):
    # level boundaries and sizes as in the reference's table: factor = 0.2 / entries of the level, 0 below 6144
    w = np.ones(30000, np.float32)
    g = oracle.weight_decay_grads(w)
    assert (g[:6144] == 0).all()
    np.testing.assert_allclose(g[6144:22528], 0.2 / (22528 - 6144), rtol=1e-6)
    np.testing.assert_allclose(g[22528:], 0.2 / (153600 - 22528), rtol=1e-6)
    top = oracle.weight_decay_grads(np.full(4, 2.0, np.float32), offset=177362944 - 2)
    np.testing.assert_allclose(top, [2 * 0.2 / (177362944 - 143808512)] * 2 + [2 * 0.2 / (210917376 - 177362944)] * 2, rtol=1e-6)


def test_cauchy_loss_against_torch(oracle):
    rng = np.random.default_rng(3)
    a, b = rng.normal(size=5000).astype(np.float32), rng.normal(size=5000).astype(np.float32)
    at = torch.tensor(a.astype(np.float64), requires_grad=True)
    loss = torch.log1p(12.5 * (at - torch.tensor(b.astype(np.float64))) ** 2).mean()
    np.testing.assert_allclose(oracle.cauchy_loss(a, b).astype(np.float64).sum(), loss.item(), rtol=1e-5)
    loss.backward()
    np.testing.assert_allclose(oracle.cauchy_loss_backward(1.0, a, b), at.grad.numpy(), rtol=1e-5, atol=1e-10)
