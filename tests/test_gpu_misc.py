"""GPU parity of the element-wise operators against the oracle (float tolerance 1e-6: the device's exp / expm1 /
sqrt and numpy's agree to a few ulp; the contraction is bit-exact where only IEEE operations are involved)."""
import numpy as np
import pytest
import torch

from inpc_amd import feature_to_opacity, spherical_contraction
from tests import helpers as H

pytestmark = pytest.mark.gpu


def test_spherical_contraction(gpu, oracle):
    rng = np.random.default_rng(0)
    p = (rng.normal(size=(300001, 3)) * rng.choice([0.2, 1.0, 5.0, 100.0], size=(300001, 1))).astype(np.float32)
    out = spherical_contraction(H.dev(p)).cpu().numpy()
    ref = oracle.spherical_contraction(p)
    np.testing.assert_array_equal(out.view(np.uint32), ref.view(np.uint32))   # +, *, /, sqrt, max only: IEEE exact
    assert spherical_contraction(torch.empty((0, 3), device=gpu)).shape == (0, 3)


def test_feature_to_opacity_forward_and_backward(gpu, oracle):
    x = np.concatenate([np.linspace(-20, 6, 100003), [-30.0, 20.0]]).astype(np.float32)
    xt = H.dev(x).requires_grad_(True)
    y = feature_to_opacity(xt)
    np.testing.assert_allclose(y.detach().cpu().numpy(), oracle.feature_to_opacity(x), rtol=1e-6, atol=1e-12)
    g = np.random.default_rng(2).normal(size=x.shape).astype(np.float32)
    y.backward(H.dev(g))
    # exp(-exp(x)) turns a relative error r of the inner exponential into exp(x) * r: up to 400 * 1e-7 at x = 6
    np.testing.assert_allclose(xt.grad.cpu().numpy(), oracle.feature_to_opacity_backward(g, x), rtol=1e-4, atol=1e-30)
    small = x <= 1.0
    np.testing.assert_allclose(xt.grad.cpu().numpy()[small], oracle.feature_to_opacity_backward(g, x)[small], rtol=2e-6,
                               atol=1e-30)


def test_weight_decay_grads(gpu, oracle):
    from inpc_amd import add_normalized_weight_decay_grads, compute_normalized_weight_decay_grads

    rng = np.random.default_rng(4)
    w = rng.normal(size=1_300_000).astype(np.float32)      # spans the levels that start at 6144 .. 1202176
    g = compute_normalized_weight_decay_grads(H.dev(w)).cpu().numpy()
    ref = oracle.weight_decay_grads(w)
    np.testing.assert_array_equal(g.view(np.uint32), ref.view(np.uint32))
    param = torch.nn.Parameter(H.dev(w))
    g0 = rng.normal(size=w.shape).astype(np.float32)
    param.grad = H.dev(g0)
    add_normalized_weight_decay_grads(param)
    np.testing.assert_array_equal(param.grad.cpu().numpy(), g0 + ref)


def test_fused_cauchy_loss(gpu, oracle):
    from inpc_amd import fused_cauchy_loss

    rng = np.random.default_rng(5)
    a, b = rng.random((3, 64, 80)).astype(np.float32), rng.random((3, 64, 80)).astype(np.float32)
    at = H.dev(a).requires_grad_(True)
    loss = fused_cauchy_loss(at, H.dev(b))
    assert loss.item() == pytest.approx(float(oracle.cauchy_loss(a, b).astype(np.float64).sum()), rel=1e-5)
    (loss * 3.0).backward()
    np.testing.assert_allclose(at.grad.cpu().numpy(), oracle.cauchy_loss_backward(3.0, a, b), rtol=2e-6, atol=1e-12)
    with pytest.raises(ValueError):
        fused_cauchy_loss(at, H.dev(b[:2]))
