"""HIP path vs the CPU checker on identical seeded inputs, through the C ABI.

Tolerance (north star): fp32 outputs and gradients within rtol 1e-5 /
atol 1e-5 * sqrt(fan_in); output shapes and valid-index masks bit-exact.
float64 runs use 1e-10.
"""
import itertools

import numpy as np
import pytest
import torch

import mconv
import _mellin_hip as hip
from _gpu import assert_close, dev, to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

VARIANTS = ["generic", None]


@pytest.fixture(params=VARIANTS, ids=["generic", "auto"])
def variant(request):
    hip.set_variant(request.param)
    yield request.param
    hip.set_variant(None)


KIND = {"mcorrlcorr": (hip.AX_MCORR, hip.AX_LCORR), "mconvlconv": (hip.AX_MCONV, hip.AX_LCONV),
        "lcorrlcorr": (hip.AX_LCORR, hip.AX_LCORR), "lconvlconv": (hip.AX_LCONV, hip.AX_LCONV)}


def _rand_params(rng, hi=4):
    return (tuple(int(v) for v in rng.integers(1, hi, 2)), tuple(int(v) for v in rng.integers(1, hi, 2)),
            tuple(int(v) for v in rng.integers(0, hi, 2)), tuple(int(v) for v in rng.integers(1, hi, 2)))


# ---------------------------------------------------------------------------
# accumulate-into-h kernels (section 1 of the C ABI)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("op", sorted(KIND))
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_accumulate_kernels_random(op, dtype):
    rng = np.random.default_rng(21)
    for trial in range(40):
        c_out, c_in, n = (int(v) for v in rng.integers(1, 7, 3))
        nf = tuple(int(v) for v in rng.integers(1, 7, 2))
        ng = tuple(int(v) for v in rng.integers(1, 30, 2))
        nh = tuple(int(v) for v in rng.integers(1, 45, 2))
        s, d, p, u = _rand_params(rng)
        tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
        w = rng.standard_normal(c_out * c_in * nf[0] * nf[1]).astype(dtype)
        x = rng.standard_normal(n * c_in * ng[0] * ng[1]).astype(dtype)
        h0 = rng.standard_normal(n * c_out * nh[0] * nh[1]).astype(dtype)
        exp = h0.copy()
        oracle.kernel2d(KIND[op], w, x, exp, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        h = to_gpu(h0)
        hip.accumulate(op, to_gpu(w), to_gpu(x), h, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        assert_close(h, exp, c_in * nf[0] * nf[1], "%s trial %d %s" % (op, trial, (nf, ng, nh, s, d, p, u, tf, tg, th)), dtype)
        # untouched outputs are bit-identical to what the caller put there
        untouched = exp == h0
        np.testing.assert_array_equal(to_np(h)[untouched], h0[untouched])


@pytest.mark.parametrize("kind", ["mcorr1d", "mconv1d"])
def test_accumulate_kernels_1d_random(kind):
    rng = np.random.default_rng(22)
    k = hip.AX_MCORR if kind == "mcorr1d" else hip.AX_MCONV
    for trial in range(40):
        c_out, c_in, n = (int(v) for v in rng.integers(1, 9, 3))
        nf, ng, nh = int(rng.integers(1, 17)), int(rng.integers(1, 300)), int(rng.integers(1, 400))
        s, d, u = (int(v) for v in rng.integers(1, 5, 3))
        p = int(rng.integers(0, 5))
        tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
        w = rng.standard_normal(c_out * c_in * nf).astype(np.float32)
        x = rng.standard_normal(n * c_in * ng).astype(np.float32)
        exp = np.zeros(n * c_out * nh, dtype=np.float32)
        oracle.kernel1d(k, w, x, exp, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        h = torch.zeros(exp.shape, device=dev())
        hip.accumulate(kind, to_gpu(w), to_gpu(x), h, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        assert_close(h, exp, c_in * nf, "%s trial %d" % (kind, trial))


def test_transposed_views_follow_reference_layout_rule():
    """.transpose(0, 1) views are used where they lie (ext/torch.cpp:40-52)."""
    rng = np.random.default_rng(23)
    x = rng.standard_normal((5, 3, 20, 7)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 2)).astype(np.float32)
    exp = oracle.mcorrlcorr(x, w, None, (1, 1), (2, 1), (1, 1), (1, 1), (1, 0))
    xt = to_gpu(np.ascontiguousarray(x.swapaxes(0, 1))).transpose(0, 1)     # (5,3,..) view of (3,5,..) memory
    wt = to_gpu(np.ascontiguousarray(w.swapaxes(0, 1))).transpose(0, 1)
    assert not xt.is_contiguous() and not wt.is_contiguous()
    got = mconv._raw_mcorrlcorr(xt, wt, None, (1, 1), (2, 1), (1, 1), (1, 1), (1, 0))
    assert_close(got, exp, 3 * 3 * 2, "transposed views")
    sliced = to_gpu(np.repeat(x, 2, axis=3))[..., ::2]                     # neither layout: copied
    got = mconv._raw_mcorrlcorr(sliced, to_gpu(w), None, (1, 1), (2, 1), (1, 1), (1, 1), (1, 0))
    assert_close(got, exp, 3 * 3 * 2, "strided input")


# ---------------------------------------------------------------------------
# operator level: forward + both gradients
# ---------------------------------------------------------------------------
def _run_op(op, x, w, b, s, d, p, u, r, go=None):
    xt = to_gpu(x).requires_grad_(True)
    wt = to_gpu(w).requires_grad_(True)
    bt = None if b is None else to_gpu(b).requires_grad_(True)
    out = getattr(mconv, "_ext_" + op)(xt, wt, bt, s, d, p, u, r)
    if go is None:
        return out, None, None, None
    out.backward(to_gpu(go))
    return out, xt.grad, wt.grad, None if bt is None else bt.grad


@pytest.mark.parametrize("op", ["mcorrlcorr", "lcorrlcorr"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_operator_random(op, dtype, variant):
    rng = np.random.default_rng(31)
    checked = 0
    for trial in range(30):
        n, c_in, c_out = (int(v) for v in rng.integers(1, 9, 3))
        nf = tuple(int(v) for v in rng.integers(1, 6, 2))
        ng = tuple(int(v) for v in rng.integers(4, 40, 2))
        s, d, p, u = _rand_params(rng)
        if trial % 3 == 0:
            u = (1, 1)                                   # what the public wrappers pass
        r = tuple(int(v) for v in rng.integers(0, 4, 2))
        x = rng.standard_normal((n, c_in) + ng).astype(dtype)
        w = rng.standard_normal((c_out, c_in) + nf).astype(dtype)
        b = rng.standard_normal(c_out).astype(dtype) if trial % 2 else None
        exp = getattr(oracle, op)(x, w, b, s, d, p, u, r)
        if exp.size == 0:
            continue
        go = rng.standard_normal(exp.shape).astype(dtype)
        gi, gw, gb = getattr(oracle, op + "_backward")(x, w, go, s, d, p, u)
        out, xg, wg, bg = _run_op(op, x, w, b, s, d, p, u, r, go)
        tag = "%s trial %d nf=%s ng=%s s=%s d=%s p=%s u=%s r=%s" % (op, trial, nf, ng, s, d, p, u, r)
        assert tuple(out.shape) == exp.shape, tag
        assert_close(out, exp, c_in * nf[0] * nf[1], "out " + tag, dtype)
        assert_close(xg, gi, c_out * nf[0] * nf[1], "grad_input " + tag, dtype)
        assert_close(wg, gw, n * exp.shape[2] * exp.shape[3], "grad_weight " + tag, dtype)
        if b is not None:
            assert_close(bg, gb, n * exp.shape[2] * exp.shape[3], "grad_bias " + tag, dtype)
        checked += 1
    assert checked >= 20


@pytest.mark.parametrize("op", ["mcorr1d", "lcorr1d"])
def test_operator_1d_random(op, variant):
    rng = np.random.default_rng(32)
    for trial in range(20):
        n, c_in, c_out = (int(v) for v in rng.integers(1, 9, 3))
        nf, ng = int(rng.integers(1, 9)), int(rng.integers(8, 200))
        s, d, u = (int(v) for v in rng.integers(1, 4, 3))
        p, r = int(rng.integers(0, 4)), int(rng.integers(0, 5))
        x = rng.standard_normal((n, c_in, ng)).astype(np.float32)
        w = rng.standard_normal((c_out, c_in, nf)).astype(np.float32)
        b = rng.standard_normal(c_out).astype(np.float32)
        if op == "mcorr1d":
            exp = oracle.mcorr1d(x, w, b, s, d, p, u, r)
            if exp.size == 0:
                continue
            go = rng.standard_normal(exp.shape).astype(np.float32)
            gi, gw, gb = oracle.mcorr1d_backward(x, w, go, s, d, p, u)
        else:
            e4 = oracle.lcorrlcorr(x[..., None], w[..., None], b, (s, 1), (d, 1), (p, 0), (u, 1), (r, 0))
            if e4.size == 0:
                continue
            exp = e4[..., 0]
            go = rng.standard_normal(exp.shape).astype(np.float32)
            gi, gw, gb = oracle.lcorrlcorr_backward(x[..., None], w[..., None], go[..., None],
                                                    (s, 1), (d, 1), (p, 0), (u, 1))
            gi, gw = gi[..., 0], gw[..., 0]
        out, xg, wg, bg = _run_op(op, x, w, b, s, d, p, u, r, go)
        tag = "%s trial %d" % (op, trial)
        assert_close(out, exp, c_in * nf, "out " + tag)
        assert_close(xg, gi, c_out * nf, "grad_input " + tag)
        assert_close(wg, gw, n * exp.shape[2], "grad_weight " + tag)
        assert_close(bg, gb, n * exp.shape[2], "grad_bias " + tag)


def test_valid_index_mask_bit_exact(variant):
    """Recover the (output, filter) -> signal index map from the kernel itself and compare
    it, bit for bit, with the checker's map: a one-hot filter at tap fx applied to the
    signal g[j] = j + 1 returns (source index + 1) wherever a tap exists and 0 elsewhere."""
    for nf, ng, s, d, p, u, extra in [(8, 512, 1, 1, 0, 1, 0), (16, 256, 1, 1, 0, 1, 5), (8, 780, 2, 2, 3, 1, 9),
                                      (5, 97, 3, 2, 4, 3, 20), (4, 64, 1, 3, 5, 2, 3)]:
        nh = mconv.mcorr_support_size(nf, ng, s, d, p, u) + extra
        sig = torch.arange(1, ng + 1, device=dev(), dtype=torch.float32).view(1, 1, ng)
        filt = torch.eye(nf, device=dev()).view(nf, 1, nf)            # channel fx = one-hot at fx
        r = nh - mconv.mcorr_valid_size(nf, ng, s, d, p, u)
        got = mconv._ext_mcorr1d(sig, filt, None, s, d, p, u, r)[0]   # (nf, nh)
        got_map = to_np(got).T.astype(np.int64) - 1
        np.testing.assert_array_equal(got_map, oracle.tap_map(oracle.AX_MCORR, nf, ng, nh, s, d, p, u))
    # linear axis
    for nf, ng, s, d, p, u in [(4, 41, 1, 1, 0, 1), (3, 41, 1, 1, 1, 1), (5, 60, 2, 3, 4, 1), (3, 30, 3, 2, 5, 2)]:
        nh = mconv.lcorr_support_size(nf, ng, s, d, p, u) + 2
        sig = torch.arange(1, ng + 1, device=dev(), dtype=torch.float32).view(1, 1, ng)
        filt = torch.eye(nf, device=dev()).view(nf, 1, nf)
        r = nh - mconv.lcorr_valid_size(nf, ng, s, d, p, u)
        got = mconv._ext_lcorr1d(sig, filt, None, s, d, p, u, r)[0]
        np.testing.assert_array_equal(to_np(got).T.astype(np.int64) - 1,
                                      oracle.tap_map(oracle.AX_LCORR, nf, ng, nh, s, d, p, u))


def test_weight_gradient_is_run_to_run_deterministic(variant):
    torch.manual_seed(5)
    x = torch.randn(8, 3, 200, 41, device=dev())
    w = torch.randn(16, 3, 8, 4, device=dev(), requires_grad=True)
    grads = []
    for _ in range(5):
        out = mconv.mcorrlcorr(x, w)
        g, = torch.autograd.grad(out, w, torch.ones_like(out))
        grads.append(g.clone())
    for g in grads[1:]:
        assert torch.equal(g, grads[0])


def test_module_trains(variant):
    """tests/test_mconv.py:776-811 of the reference: gradients reach weight and bias."""
    torch.manual_seed(30)
    layer = mconv.MCorr1d(40, 30, 5).to(dev())
    inp = torch.rand(50, 40, 20, requires_grad=True, device=dev())
    layer(inp).sum().backward()
    assert layer.bias.grad.abs().sum() > 0 and layer.weight.grad.abs().sum() > 0
    layer2 = mconv.MCorrLCorr(12, 11, (10, 9)).to(dev())
    ins = torch.randn(13, 12, 15, 14, requires_grad=True, device=dev())
    loss = torch.nn.MSELoss()(layer2(ins).sum((1, 2, 3)), torch.randn(13, device=dev()))
    loss.backward()
    assert layer2.bias.grad.abs().sum() > 0 and layer2.weight.grad.abs().sum() > 0
    assert ins.grad is not None and ins.grad.shape == ins.shape


@pytest.mark.parametrize("shape", [((6, 3, 3, 4), (10, 3, 5, 5)), ((4, 1, 5, 4), (6, 1, 2, 2))])
def test_gradcheck_float64(shape):
    """tests/test_mconv.py:686-729 of the reference, on the device in float64."""
    torch.manual_seed(1)
    f_shape, g_shape = shape
    for s, d, p, u in itertools.product([1, 2], [1, 2], [3, 4], [1, 2]):
        f = torch.rand(f_shape, dtype=torch.double, device=dev(), requires_grad=True)
        g = torch.rand(g_shape, dtype=torch.double, device=dev(), requires_grad=True)
        b = torch.rand(f_shape[:1], dtype=torch.double, device=dev(), requires_grad=True)
        torch.autograd.gradcheck(
            lambda g, f, b: mconv._ext_mcorrlcorr(g, f, b, (s, s), (d, d), (p, p), (u, u), (p, p)),
            (g, f, b), atol=1e-6)
