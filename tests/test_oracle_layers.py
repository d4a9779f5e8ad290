"""The CPU checker's pointwise layers (log compression, dilation lift) against what
pins them without the reference: PyTorch's own elementwise routines and autograd on the
CPU (the reference composes exactly those, layers.py:8-21 and 100-101), closed forms,
and finite differences."""
import numpy as np
import pytest
import torch

from oracle import oracle


def _torch_pair(x, eps, tau, dim):
    """The reference's composition, written with PyTorch CPU ops in float64."""
    y = x
    if eps is not None:
        y = (y.abs() + eps).log()
    if tau is not None:
        shape = [1] * y.dim()
        shape[dim] = y.shape[dim]
        y = y * (torch.arange(1, y.shape[dim] + 1, dtype=y.dtype) ** tau).reshape(shape)
    return y


@pytest.mark.parametrize("use_eps,use_tau", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("dim", [0, 1, 2, -1])
def test_values_and_gradients_match_pytorch_cpu(use_eps, use_tau, dim):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 5, 4))
    x[0, 0, 0] = 0.0                                     # |x| at 0
    g = rng.standard_normal(x.shape)
    eps, tau = (0.37 if use_eps else None), (1.3 if use_tau else None)
    d = dim % 3
    xt = torch.tensor(x, requires_grad=True)
    et = torch.tensor(eps, dtype=torch.float64, requires_grad=True) if use_eps else None
    tt = torch.tensor(tau, dtype=torch.float64, requires_grad=True) if use_tau else None
    yt = _torch_pair(xt, et, tt, d)
    yt.backward(torch.tensor(g))
    np.testing.assert_allclose(oracle.log_lift(x, eps, tau, d), yt.detach().numpy(), rtol=1e-13, atol=1e-13)
    gx, ge, gt = oracle.log_lift_backward(x, g, eps, tau, d)
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    if use_eps:
        assert abs(ge - float(et.grad)) <= 1e-11 * max(1.0, abs(ge))
    else:
        assert ge == 0.0
    if use_tau:
        assert abs(gt - float(tt.grad)) <= 1e-11 * max(1.0, abs(gt))
    else:
        assert gt == 0.0


def test_closed_forms():
    x = np.linspace(-2.0, 2.0, 24).reshape(2, 4, 3)
    # tau = 0: the lift is the identity; tau = 1: multiplication by t = 1 .. T
    np.testing.assert_allclose(oracle.log_lift(x, None, 0.0, 1), x)
    np.testing.assert_allclose(oracle.log_lift(x, None, 1.0, 1), x * np.arange(1, 5).reshape(1, 4, 1))
    np.testing.assert_allclose(oracle.log_lift(x, None, 2.0, 2), x * (np.arange(1, 4) ** 2).reshape(1, 1, 3))
    # log compression: even in x, log(eps) at 0, log(eps + 1) at +-1
    np.testing.assert_allclose(oracle.log_lift(x, 0.5, None), oracle.log_lift(-x, 0.5, None))
    np.testing.assert_allclose(oracle.log_lift(np.array([[[0.0, 1.0, -1.0]]]), 0.5, None),
                               [[[np.log(0.5), np.log(1.5), np.log(1.5)]]])


def test_finite_differences():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 6, 3)) + 0.1
    g = rng.standard_normal(x.shape)
    eps, tau, h = 0.8, 0.6, 1e-6
    gx, ge, gt = oracle.log_lift_backward(x, g, eps, tau, 1)
    f = lambda x_, e_, t_: float((oracle.log_lift(x_, e_, t_, 1) * g).sum())
    assert abs((f(x, eps + h, tau) - f(x, eps - h, tau)) / (2 * h) - ge) < 1e-6
    assert abs((f(x, eps, tau + h) - f(x, eps, tau - h)) / (2 * h) - gt) < 1e-6
    for idx in [(0, 0, 0), (1, 5, 2), (0, 3, 1)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        assert abs((f(xp, eps, tau) - f(xm, eps, tau)) / (2 * h) - gx[idx]) < 1e-6
