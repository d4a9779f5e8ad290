"""Parity at the BASELINE configurations (seeded as the measurement plan states):
HIP path vs the CPU checker, through the module API and hence the C ABI.

Where the checker would need minutes at full size it is run on slices that the
structure of the operator makes exact: outputs are independent across batch
elements and output channels, input gradients across batch elements, weight
gradients across (c_out, c_in) pairs.  Full-size runs are additionally checked
through size-independent identities (adjointness, linearity)."""
import numpy as np
import pytest
import torch

import mconv
import _mellin_hip as hip
from _gpu import assert_close, dev, f64, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["generic", None], ids=["generic", "auto"])
def variant(request):
    hip.set_variant(request.param)
    yield request.param
    hip.set_variant(None)


def _uniform(gen, shape, bound):
    return (torch.rand(shape, generator=gen) * 2 - 1) * bound


def test_cfg1_mcorr1d_forward(variant):
    """N=8, C_in=3, C_out=16, length 256, kernel 16, s=d=u=1, p=0; seed 0."""
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(8, 3, 256, generator=gen)
    w = _uniform(gen, (16, 3, 16), 48 ** -0.5)
    out = mconv.mcorr1d(x.to(dev()), w.to(dev()))
    assert tuple(out.shape) == (8, 16, 16)
    assert_close(out, oracle.mcorr1d(x.numpy(), w.numpy()), 48, "cfg1")
    # the registered convolution op on the same tensors: output length 256
    outc = mconv._ext_mconv1d(x.to(dev()), w.to(dev()))
    assert tuple(outc.shape) == (8, 16, 256)
    assert_close(outc, oracle.mconv1d(x.numpy(), w.numpy()), 48, "cfg1 mconv1d")


@pytest.mark.parametrize("s", [1, 2])
@pytest.mark.parametrize("d", [1, 2])
@pytest.mark.parametrize("p", [0, 3])
def test_cfg2_1d_forward_backward(s, d, p, variant):
    """N=32, C_in=41, C_out=128, lengths U[100,780] zero-padded to 780, kernel 8; seed 1."""
    gen = torch.Generator().manual_seed(1)
    n, c_in, c_out, L, k = 32, 41, 128, 780, 8
    x = torch.randn(n, c_in, L, generator=gen)
    lens = torch.randint(100, 781, (n,), generator=gen)
    x = x * (torch.arange(L)[None, None, :] < lens[:, None, None])
    bound = (c_in * k) ** -0.5
    w, b = _uniform(gen, (c_out, c_in, k), bound), _uniform(gen, (c_out,), bound)
    for op in ("mcorr1d", "lcorr1d"):
        # the GPU runs all 32 utterances of both layer kinds; for the linear one (eight times the
        # outputs) the checker covers the output and the input gradient of the first 8 utterances
        # and the weight / bias gradients (sums over the whole batch) of the first 16 channels
        xt = x.to(dev()).requires_grad_(True)
        wt, bt = w.to(dev()).requires_grad_(True), b.to(dev()).requires_grad_(True)
        out = getattr(mconv, op)(xt, wt, bt, s, d, p)
        go = torch.randn(out.shape, generator=gen)
        out.backward(go.to(dev()))
        tag = "cfg2 %s s=%d d=%d p=%d" % (op, s, d, p)
        if op == "mcorr1d":
            exp = oracle.mcorr1d(x.numpy(), w.numpy(), b.numpy(), s, d, p)
            gi, gw, gb = oracle.mcorr1d_backward(*f64(x.numpy(), w.numpy(), go.numpy()), s, d, p)
            nb, mc = n, c_out
        else:
            nb, mc = 8, 16
            xs = x[:nb].numpy()
            exp = oracle.lcorrlcorr(xs[..., None], w.numpy()[..., None], b.numpy(), (s, 1), (d, 1), (p, 0))[..., 0]
            gi, _, _ = oracle.lcorrlcorr_backward(*f64(xs[..., None], w.numpy()[..., None],
                                                       go[:nb].numpy()[..., None]), (s, 1), (d, 1), (p, 0))
            _, gw, gb = oracle.lcorrlcorr_backward(*f64(x.numpy()[..., None], w[:mc].numpy()[..., None],
                                                        go[:, :mc].contiguous().numpy()[..., None]), (s, 1), (d, 1), (p, 0))
            gi, gw = gi[..., 0], gw[..., 0]
        assert tuple(out.shape[:2]) == (n, c_out)
        assert_close(out[:nb], exp, c_in * k, tag + " out")
        assert_close(xt.grad[:nb], gi, c_out * k, tag + " grad_input")
        assert_close(wt.grad[:mc], gw, n * exp.shape[2], tag + " grad_weight")
        assert_close(bt.grad[:mc], gb, n * exp.shape[2], tag + " grad_bias")


def _cfg3(gen):
    x = torch.randn(32, 3, 512, 41, generator=gen)
    bound = 96 ** -0.5
    return x, _uniform(gen, (64, 3, 8, 4), bound), _uniform(gen, (64,), bound)


def test_cfg3_mconv2d_forward_backward(variant):
    """N=32, C_in=3, 512 x 41, C_out=64, kernel 8 x 4; seed 2.  Full size on both sides."""
    gen = torch.Generator().manual_seed(2)
    x, w, b = _cfg3(gen)
    xt = x.to(dev()).requires_grad_(True)
    wt, bt = w.to(dev()).requires_grad_(True), b.to(dev()).requires_grad_(True)
    out = mconv.mcorrlcorr(xt, wt, bt)
    assert tuple(out.shape) == (32, 64, 64, 38)
    go = torch.randn(out.shape, generator=gen)
    out.backward(go.to(dev()))
    exp = oracle.mcorrlcorr(x.numpy(), w.numpy(), b.numpy())
    gi, gw, gb = oracle.mcorrlcorr_backward(*f64(x.numpy(), w.numpy(), go.numpy()))
    assert_close(out, exp, 96, "cfg3 out")
    assert_close(xt.grad, gi, 64 * 32, "cfg3 grad_input")
    assert_close(wt.grad, gw, 32 * 64 * 38, "cfg3 grad_weight")
    assert_close(bt.grad, gb, 32 * 64 * 38, "cfg3 grad_bias")
    # only 269 of the 512 input rows feed any output: the others get exactly zero gradient
    touched = np.unique(oracle.tap_map(oracle.AX_MCORR, 8, 512, 64))
    touched = touched[touched >= 0]
    mask = np.ones(512, bool)
    mask[touched] = False
    assert len(touched) == 269 and not to_np(xt.grad)[:, :, mask].any()


def test_cfg3_lconv2d_forward_backward(variant):
    """The same batch through the linear x linear layer (output 505 x 38); checker on slices."""
    gen = torch.Generator().manual_seed(2)
    x, w, b = _cfg3(gen)
    xt = x.to(dev()).requires_grad_(True)
    wt, bt = w.to(dev()).requires_grad_(True), b.to(dev()).requires_grad_(True)
    out = mconv.lcorrlcorr(xt, wt, bt)
    assert tuple(out.shape) == (32, 64, 505, 38)
    go = torch.randn(out.shape, generator=gen)
    out.backward(go.to(dev()))
    xn, wn, bn, gon = x.numpy(), w.numpy(), b.numpy(), go.numpy()
    nb = [0, 17, 31]
    exp = oracle.lcorrlcorr(xn[nb], wn, bn)
    assert_close(out[nb], exp, 96, "cfg3-l out")
    gi, _, _ = oracle.lcorrlcorr_backward(xn[nb], wn, gon[nb])
    assert_close(xt.grad[nb], gi, 64 * 32, "cfg3-l grad_input")
    co = [0, 13, 63]
    _, gw, gb = oracle.lcorrlcorr_backward(*f64(xn, wn[co], np.ascontiguousarray(gon[:, co])))
    assert_close(wt.grad[co], gw, 32 * 505 * 38, "cfg3-l grad_weight")
    assert_close(bt.grad[co], gb, 32 * 505 * 38, "cfg3-l grad_bias")


def test_cfg4_lconv2d_wide_channels(variant):
    """N=32, C_in=128, C_out=256, 256 x 41, kernel 3 x 3, d=(2,1), p=(2,1); seed 3."""
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(32, 128, 256, 41, generator=gen)
    bound = 1152 ** -0.5
    w, b = _uniform(gen, (256, 128, 3, 3), bound), _uniform(gen, (256,), bound)
    s, d, p = (1, 1), (2, 1), (2, 1)
    xt = x.to(dev()).requires_grad_(True)
    wt, bt = w.to(dev()).requires_grad_(True), b.to(dev()).requires_grad_(True)
    out = mconv.lcorrlcorr(xt, wt, bt, s, d, p)
    assert tuple(out.shape) == (32, 256, 254, 40)
    go = torch.randn(out.shape, generator=gen)
    out.backward(go.to(dev()))
    xn, wn, bn, gon = x.numpy(), w.numpy(), b.numpy(), go.numpy()
    # forward: 2 utterances x 16 output channels
    nb, co = [3, 30], list(range(0, 256, 16))
    exp = oracle.lcorrlcorr(xn[nb], wn[co], bn[co], s, d, p)
    assert_close(out[nb][:, co], exp, 1152, "cfg4 out")
    # input gradient: one utterance, all channels
    gi, _, _ = oracle.lcorrlcorr_backward(xn[5:6], wn, gon[5:6], s, d, p)
    assert_close(xt.grad[5:6], gi, 256 * 9, "cfg4 grad_input")
    # weight gradient: 4 x 6 channel pairs over the whole batch
    co, ci = [0, 77, 128, 255], [0, 1, 31, 64, 100, 127]
    _, gw, _ = oracle.lcorrlcorr_backward(*f64(np.ascontiguousarray(xn[:, ci]), wn[co][:, ci],
                                               np.ascontiguousarray(gon[:, co])), s, d, p)
    assert_close(wt.grad[co][:, ci], gw, 32 * 254 * 40, "cfg4 grad_weight")
    # against the vendor library on the whole tensor (torch conv2d = MIOpen), as a second opinion
    with torch.no_grad():
        lib_out = torch.nn.functional.conv2d(torch.nn.functional.pad(xt, (1, 0, 2, 0)), wt, bt, dilation=d)
    assert lib_out.shape == out.shape
    torch.testing.assert_close(out, lib_out, rtol=1e-4, atol=1e-4 * 1152 ** 0.5)


def test_full_size_identities(variant):
    """Size-independent properties at the full cfg3 size: bilinearity and adjointness."""
    gen = torch.Generator().manual_seed(7)
    x, w, _ = _cfg3(gen)
    x2 = torch.randn(x.shape, generator=gen)
    xt, x2t, wt = x.to(dev()), x2.to(dev()), w.to(dev())
    for op in (mconv.mcorrlcorr, mconv.lcorrlcorr):
        a, b2 = op(xt, wt), op(x2t, wt)
        ab = op(xt * 0.5 + x2t * 2.0, wt)
        torch.testing.assert_close(ab, a * 0.5 + b2 * 2.0, rtol=1e-4, atol=1e-4)
        xg = xt.clone().requires_grad_(True)
        wg = wt.clone().requires_grad_(True)
        out = op(xg, wg)
        y = torch.randn(out.shape, generator=gen).to(dev())
        out.backward(y)
        lhs = float((out.double() * y.double()).sum())
        # <fwd(x; w), y> = <x, grad_input> = <w, grad_weight>
        for other in (float((xg.double() * xg.grad.double()).sum()), float((wg.double() * wg.grad.double()).sum())):
            assert abs(other - lhs) <= 1e-4 * abs(lhs) + 1.0, (op.__name__, lhs, other)
