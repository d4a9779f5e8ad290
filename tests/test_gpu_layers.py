"""Log compression and dilation lift on the GPU, through the C ABI, against the CPU
checker: values, input gradients and the two parameter gradients.

Tolerance: fp32 values and input gradients rtol 1e-5 / atol 1e-5 times the largest
lift factor T ** tau (the logarithm's rounding error of a few 1e-8 is multiplied by
it, in any fp32 evaluation); the parameter
gradients are sums over every element and are compared, like the weight gradients,
with the checker evaluated in float64, rtol 1e-5 / atol 1e-5 * sqrt(number of terms).
float64 runs are held to 1e-12.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
import layers
from _gpu import to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

SHAPES = [((6, 16, 41), 1), ((3, 7), 0), ((2, 3, 5, 4), 2), ((4, 25, 1), -2), ((1, 1, 1), 1), ((5, 300), -1),
          ((70, 40, 41), 1)]


def _tol(dtype, terms=1):
    return (1e-5, 1e-5 * terms ** 0.5) if dtype == np.float32 else (1e-12, 1e-12 * terms ** 0.5)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("mode", ["log", "lift", "both"])
@pytest.mark.parametrize("shape,dim", SHAPES, ids=[str(s[0]) for s in SHAPES])
def test_c_abi_matches_checker(shape, dim, mode, dtype):
    rng = np.random.default_rng(abs(hash((shape, dim, mode))) % 2 ** 31)
    x = rng.standard_normal(shape).astype(dtype)
    x.flat[0] = 0.0
    g = rng.standard_normal(shape).astype(dtype)
    eps = 0.41 if mode != "lift" else None
    tau = 1.37 if mode != "log" else None
    flags = (hip.PW_LOG if eps is not None else 0) | (hip.PW_LIFT if tau is not None else 0)
    d = dim % len(shape)
    outer, t, inner = int(np.prod(shape[:d], dtype=np.int64)), shape[d], int(np.prod(shape[d + 1:], dtype=np.int64))
    xg, gg = to_gpu(x), to_gpu(g)
    y = torch.full_like(xg, float("nan"))
    hip.log_lift_forward(xg, eps or 1.0, tau or 0.0, flags, outer, t, inner, y)
    rtol, atol = _tol(dtype)
    atol *= float(t) ** (tau or 0.0)
    np.testing.assert_allclose(to_np(y), oracle.log_lift(x, eps, tau, d), rtol=rtol, atol=atol)
    gx = torch.full_like(xg, float("nan"))
    gp = torch.full((2,), float("nan"), dtype=xg.dtype, device=xg.device)
    hip.log_lift_backward(xg, gg, eps or 1.0, tau or 0.0, flags, outer, t, inner, gx, gp)
    ex, ee, et = oracle.log_lift_backward(x, g, eps, tau, d)
    np.testing.assert_allclose(to_np(gx), ex, rtol=rtol, atol=atol / (eps or 1.0))
    rtol, atol = _tol(dtype, x.size)
    got = to_np(gp)
    # scale of the sums' terms: grad_y / (eps + |x|) reaches 1 / eps
    scale = max(1.0, 1.0 / (eps or 1.0)) * max(1.0, np.log(max(t, 2)) * float(t) ** (tau or 0.0))
    assert abs(got[0] - ee) <= rtol * abs(ee) + atol * scale, (got[0], ee)
    assert abs(got[1] - et) <= rtol * abs(et) + atol * scale, (got[1], et)


def test_modules_train_like_the_reference_composition():
    """The modules (log_eps / log_tau parameters, exp inside forward) against the same
    composition written with PyTorch ops in float64 on the CPU."""
    torch.manual_seed(11)
    x = torch.randn(9, 20, 41, device="cuda")
    fused = layers.LogCompressionLift(dim=1).cuda()
    lc, dl = layers.LogCompression().cuda(), layers.DilationLift(dim=1).cuda()
    with torch.no_grad():
        fused.log_eps.fill_(-0.5)                        # eps = 0.61, tau = 1.22: well-conditioned sums
        fused.log_tau.fill_(0.2)
        lc.log_eps.copy_(fused.log_eps)
        dl.log_tau.copy_(fused.log_tau)
    g = torch.randn_like(x)
    xa = x.clone().requires_grad_(True)
    ya = fused(xa)
    ya.backward(g)
    xb = x.clone().requires_grad_(True)
    yb = dl(lc(xb))
    yb.backward(g)
    # CPU float64 composition with autograd
    xc = x.double().cpu().requires_grad_(True)
    le = fused.log_eps.detach().double().cpu().requires_grad_(True)
    lt = fused.log_tau.detach().double().cpu().requires_grad_(True)
    yc = (xc.abs() + le.exp()).log() * (torch.arange(1, 21, dtype=torch.float64) ** lt.exp()).reshape(1, 20, 1)
    yc.backward(g.double().cpu())
    for y_, x_, pe, pt in ((ya, xa, fused.log_eps, fused.log_tau), (yb, xb, lc.log_eps, dl.log_tau)):
        lift = 20.0 ** float(lt.exp())
        np.testing.assert_allclose(to_np(y_), yc.detach().numpy(), rtol=1e-5, atol=1e-5 * lift)
        np.testing.assert_allclose(to_np(x_.grad), xc.grad.numpy(), rtol=1e-5, atol=1e-5 * lift / float(le.exp()))
        # sums of numel terms of size up to lift * ln(20) / eps (times the parameter itself: chain rule)
        tol = 1e-5 * x.numel() ** 0.5 * lift * 3.0 / float(le.exp()) * 2
        assert abs(float(pe.grad) - float(le.grad)) <= 1e-5 * abs(float(le.grad)) + tol
        assert abs(float(pt.grad) - float(lt.grad)) <= 1e-5 * abs(float(lt.grad)) + tol


def test_backward_is_run_to_run_deterministic():
    x = torch.randn(64, 128, 41, device="cuda")
    g = torch.randn_like(x)
    outs = []
    for _ in range(3):
        gx = torch.empty_like(x)
        gp = torch.empty(2, device="cuda")
        hip.log_lift_backward(x, g, 0.3, 0.9, hip.PW_LOG | hip.PW_LIFT, 64, 128, 41, gx, gp)
        outs.append((gx.clone(), gp.clone()))
    for gx, gp in outs[1:]:
        assert torch.equal(gx, outs[0][0]) and torch.equal(gp, outs[0][1])


def test_errors_and_edge_cases():
    x = torch.randn(4, 5, device="cuda")
    with pytest.raises(RuntimeError, match="not a valid dimension"):
        layers.dilation_lift(x, torch.tensor(1.0), 2)
    with pytest.raises(RuntimeError, match="eps must be positive"):
        hip.log_lift_forward(x, 0.0, 0.0, hip.PW_LOG, 4, 5, 1, torch.empty_like(x))
    with pytest.raises(RuntimeError, match="flags"):
        hip.log_lift_forward(x, 1.0, 0.0, 0, 4, 5, 1, torch.empty_like(x))
    with pytest.raises(RuntimeError, match="GPUs only"):
        layers.log_compression(torch.randn(3), torch.tensor(1.0))
    empty = torch.empty(0, 5, device="cuda")
    assert layers.dilation_lift(empty, torch.tensor(1.0), 1).shape == (0, 5)
    noise = layers.ScaledGaussianNoise(dim=1, eps=0.5).cuda()
    noise.eval()
    assert noise(x) is x
    noise.train()
    y = noise(x)
    assert y.shape == x.shape and not torch.equal(y, x)
    assert float((y - x).abs().max()) < 0.5 * float(x.abs().max()) * 8
