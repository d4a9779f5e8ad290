"""Bias gradient and the backward of a fused ReLU in one pass (mellin_bias_grad_f32 / _f16): the masked
gradient must be grad_out where out > 0 and zero elsewhere, exactly; the per-channel sums are
compared with float64 sums of the same values at rtol 1e-5 / atol 1e-5 * sqrt(terms) and must not
change from run to run (half tensors: fp32 sums, rounded to half once).  The reference computes both in PyTorch (ext/torch.cpp:231,300 and the
model's ReLU, models.py:423-425)."""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
import mconv

pytestmark = pytest.mark.gpu

SHAPES = [(32, 64, 505, 38), (3, 5, 7, 11), (2, 33, 4097, 1), (1, 1, 1, 1), (5, 7, 4096, 1), (4, 130, 60, 33)]


@pytest.mark.parametrize("shape", SHAPES, ids=["x".join(map(str, s)) for s in SHAPES])
@pytest.mark.parametrize("masked", [True, False], ids=["relu", "plain"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["float32", "half"])
def test_bias_grad_matches_float64_sums(shape, masked, dtype):
    torch.manual_seed(sum(shape))
    go = torch.randn(*shape, device="cuda").to(dtype)
    out = torch.relu(torch.randn(*shape, device="cuda")).to(dtype) if masked else None
    g, gb = hip.bias_grad(go, out)
    exp_g = go * (out > 0) if masked else go
    assert torch.equal(g, exp_g)
    if not masked:
        assert g.data_ptr() == go.data_ptr()                # nothing is copied
    exp = exp_g.double().sum((0, 2, 3))
    terms = shape[0] * shape[2] * shape[3]
    assert gb.dtype == dtype
    # (half: the fp32 sum rounded once, relative 2^-11)
    np.testing.assert_allclose(gb.double().cpu().numpy(), exp.cpu().numpy(), rtol=1e-5 if dtype == torch.float32 else 5e-4,
                               atol=1e-5 * terms ** 0.5)
    g2, gb2 = hip.bias_grad(go, out)
    assert torch.equal(gb, gb2) and torch.equal(g, g2)


def test_bias_grad_edge_cases():
    empty = torch.empty(0, 4, 3, 2, device="cuda")
    g, gb = hip.bias_grad(empty, None)
    assert gb.shape == (4,) and float(gb.abs().sum()) == 0.0
    go = torch.randn(2, 3, 5, 5, device="cuda")
    need = hip.lib.mellin_bias_grad_workspace(2, 3, 25)
    assert need == 2 * 3 * 4
    gb = torch.empty(3, device="cuda")
    rc = hip.lib.mellin_bias_grad_f32(hip._dp(go), None, 2, 3, 25, None, hip._dp(gb), None, 0, hip._stream(go.device))
    assert rc != 0 and "workspace" in hip.last_error()
    rc = hip.lib.mellin_bias_grad_f32(hip._dp(go), None, 70000, 3, 25, None, hip._dp(gb), None, 0,
                                      hip._stream(go.device))
    assert rc != 0 and "65535" in hip.last_error()


def test_half_layer_backward_uses_it():
    """Half tensors through autograd: the masked gradient and the bias gradient come from the
    library's pass, not from PyTorch's composition."""
    torch.manual_seed(6)
    x = torch.randn(4, 3, 40, 21, device="cuda").half()
    w = (torch.randn(16, 3, 4, 4, device="cuda") * 0.2).half().requires_grad_(True)
    b = (torch.randn(16, device="cuda") * 0.1).half().requires_grad_(True)
    y = mconv.lcorrlcorr(x, w, b, activation="relu")
    gy = torch.randn_like(y)
    gw, gb = torch.autograd.grad(y, (w, b), gy)
    masked = (gy * (y > 0)).float()
    assert gb.dtype == torch.float16 and torch.equal(gb, masked.sum((0, 2, 3)).half())
    w2, b2 = w.detach().float().requires_grad_(True), b.detach().float().requires_grad_(True)
    y2 = torch.relu(torch.nn.functional.conv2d(x.float(), w2, b2))
    gw2, = torch.autograd.grad(y2, (w2,), masked)
    torch.testing.assert_close(gw.float(), gw2, rtol=2e-3, atol=1e-4 * (4 * 37 * 18) ** 0.5)


def test_layer_backward_uses_it():
    """Through autograd: bias and fused-ReLU gradients of a layer against PyTorch's own composition."""
    torch.manual_seed(5)
    x = torch.randn(4, 3, 40, 21, device="cuda")
    w = (torch.randn(16, 3, 4, 4, device="cuda") * 0.2).requires_grad_(True)
    b = (torch.randn(16, device="cuda") * 0.1).requires_grad_(True)
    y = mconv.lcorrlcorr(x, w, b, activation="relu")
    gy = torch.randn_like(y)
    gw, gb = torch.autograd.grad(y, (w, b), gy)
    w2, b2 = w.detach().clone().requires_grad_(True), b.detach().clone().requires_grad_(True)
    y2 = torch.relu(torch.nn.functional.conv2d(x, w2, b2))
    gw2, gb2 = torch.autograd.grad(y2, (w2, b2), gy)
    torch.testing.assert_close(y, y2, rtol=1e-5, atol=1e-5 * 48 ** 0.5)
    torch.testing.assert_close(gb, gb2, rtol=1e-4, atol=1e-4 * (4 * 37 * 18) ** 0.5)
    torch.testing.assert_close(gw, gw2, rtol=1e-4, atol=1e-4 * (4 * 37 * 18) ** 0.5)


@pytest.mark.parametrize("shape", [(4, 8, 50, 38), (2, 3, 7, 41), (3, 2, 5, 2), (2, 2, 3, 1), (1, 64, 777, 38)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["float32", "half"])
def test_frequency_pool_equals_max_pool2d(shape, dtype):
    """The stack's frequency pooling (pairs of neighbouring bins): values and gradient bit for bit
    what max_pool2d(x, (1, 2)) gives, ties and an odd last column included."""
    from conv_stack import freq_max_pool
    torch.manual_seed(shape[2])
    x = torch.randn(*shape, device="cuda").to(dtype)
    x[..., : shape[3] // 2 * 2] = torch.where(torch.rand_like(x[..., : shape[3] // 2 * 2]) < 0.2,
                                              torch.zeros(()).to(x), x[..., : shape[3] // 2 * 2])   # ties at zero
    a = x.clone().requires_grad_(True)
    b = x.clone().requires_grad_(True)
    if shape[3] < 2:
        import _mellin_hip
        y, which = _mellin_hip.pool_pairs_forward(x)
        assert y.shape == shape[:3] + (0,)
        gx = _mellin_hip.pool_pairs_backward(torch.empty_like(y), which, shape[3])
        assert gx.shape == shape and float(gx.abs().sum()) == 0.0
        return
    ya, yb = freq_max_pool(a), torch.nn.functional.max_pool2d(b, (1, 2))
    assert torch.equal(ya, yb)
    g = torch.randn_like(ya)
    ya.backward(g)
    yb.backward(g)
    assert torch.equal(a.grad, b.grad)
