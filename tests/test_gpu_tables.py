"""The HIP kernels, called through the C ABI, against the reference's
known-answer tables: the same matrix as the reference's CUDA test mains
(c/tests/test_*_cuda.cc over c/tests/CMakeLists.txt:35-49)."""
import itertools

import numpy as np
import pytest
import torch

import _fixtures as fx
import _mellin_hip as hip
from _gpu import to_gpu, to_np

pytestmark = pytest.mark.gpu

FLAGS = list(itertools.product([False, True], repeat=3))
EXTRA = [-1, 0, 10]
SUP = {"mcorr": lambda c, a: _sup(hip.AX_MCORR, c, a), "mconv": lambda c, a: _sup(hip.AX_MCONV, c, a)}


def _sup(kind, c, a):
    import mconv
    fn = {hip.AX_MCORR: mconv.mcorr_support_size, hip.AX_MCONV: mconv.mconv_support_size,
          hip.AX_LCORR: mconv.lcorr_support_size, hip.AX_LCONV: mconv.lconv_support_size}[kind]
    return fn(c["nf" + a], c["ng" + a], c["s" + a], c["d" + a], c["p" + a], c["u" + a])


def _cases(*names):
    return [(n, i) for n in names for i in range(fx.num_cases(n))]


def _tol(dtype, c):
    """float64: the reference's own 1e-10; float32: rtol 1e-5 / atol 1e-5 * sqrt(fan_in)."""
    if dtype == np.float64:
        return dict(rtol=0, atol=1e-10)
    fan_in = c["c_in"] * c["nfx"] * c.get("nfy", 1)
    return dict(rtol=1e-5, atol=1e-5 * fan_in ** 0.5)


@pytest.mark.parametrize("dtype", [np.float64, np.float32], ids=["f64", "f32"])
@pytest.mark.parametrize("name,idx", _cases("mcorr1d", "mconv1d"))
def test_1d_tables(name, idx, dtype):
    c = fx.case(name, idx)
    kind = hip.AX_MCORR if name == "mcorr1d" else hip.AX_MCONV
    sup = _sup(kind, c, "x")
    for batch, (tf, tg, th), extra in itertools.product([1, 2], FLAGS, EXTRA):
        nh = sup + extra
        if nh <= 0:
            continue
        f = to_gpu(fx.filter_array(c, tf).astype(dtype))
        g = to_gpu(fx.tiled(c["G"], batch, c["c_in"], c["ngx"], 1, 0, 0, tg).astype(dtype))
        exp = fx.tiled(c["H"], batch, c["c_out"], sup, 1, extra, 0, th).astype(dtype)
        h = torch.zeros(exp.shape, dtype=f.dtype, device=f.device)
        hip.accumulate(name, f, g, h, c["c_out"], c["c_in"], batch, c["nfx"], c["ngx"], nh,
                       c["sx"], c["dx"], c["px"], c["ux"], tf, tg, th)
        np.testing.assert_allclose(to_np(h), exp, **_tol(dtype, c),
                                   err_msg="%s[%d] b=%d flags=%s extra=%d" % (name, idx, batch, (tf, tg, th), extra))


@pytest.mark.parametrize("dtype", [np.float64, np.float32], ids=["f64", "f32"])
@pytest.mark.parametrize("name,idx", _cases("mcorr1d", "lcorr1d", "mcorrlcorr",
                                            "mconv1d", "lconv1d", "mconvlconv"))
def test_2d_tables(name, idx, dtype):
    c = fx.case(name, idx)
    corr = name in ("mcorr1d", "lcorr1d", "mcorrlcorr")
    op = "mcorrlcorr" if corr else "mconvlconv"
    supx = _sup(hip.AX_MCORR if corr else hip.AX_MCONV, c, "x")
    supy = _sup(hip.AX_LCORR if corr else hip.AX_LCONV, c, "y")
    for batch, (tf, tg, th), extra in itertools.product([1, 2], FLAGS, EXTRA):
        nhx, nhy = supx + extra, supy + extra
        if nhx <= 0 or nhy <= 0:
            continue
        f = to_gpu(fx.filter_array(c, tf).astype(dtype))
        g = to_gpu(fx.tiled(c["G"], batch, c["c_in"], c["ngx"], c["ngy"], 0, 0, tg).astype(dtype))
        exp = fx.tiled(c["H"], batch, c["c_out"], supx, supy, extra, extra, th).astype(dtype)
        h = torch.zeros(exp.shape, dtype=f.dtype, device=f.device)
        hip.accumulate(op, f, g, h, c["c_out"], c["c_in"], batch, (c["nfx"], c["nfy"]),
                       (c["ngx"], c["ngy"]), (nhx, nhy), (c["sx"], c["sy"]), (c["dx"], c["dy"]),
                       (c["px"], c["py"]), (c["ux"], c["uy"]), tf, tg, th)
        np.testing.assert_allclose(to_np(h), exp, **_tol(dtype, c),
                                   err_msg="%s[%d] b=%d flags=%s extra=%d" % (name, idx, batch, (tf, tg, th), extra))


@pytest.mark.parametrize("name,idx", _cases("mcorr1d", "lcorr1d", "mcorrlcorr"))
@pytest.mark.parametrize("bias", [True, False])
def test_operator_values(name, idx, bias):
    """tests/test_mconv.py:604-623 of the reference: request r = support - valid so the
    whole support is produced, with and without a random bias."""
    import mconv
    c = fx.case(name, idx)
    supx = _sup(hip.AX_MCORR, c, "x")
    supy = _sup(hip.AX_LCORR, c, "y")
    s, d, p, u = ((c[k + "x"], c[k + "y"]) for k in "sdpu")
    w = to_gpu(fx.filter_array(c).astype(np.float32))
    x = to_gpu(fx.tiled(c["G"], 3, c["c_in"], c["ngx"], c["ngy"]).astype(np.float32))
    exp = fx.tiled(c["H"], 3, c["c_out"], supx, supy).astype(np.float32)
    b = torch.randint(-5, 5, (c["c_out"],), device=w.device).float() if bias else None
    if bias:
        exp = exp + to_np(b).reshape(1, -1, 1, 1)
    rx = supx - mconv.mcorr_valid_size(c["nfx"], c["ngx"], s[0], d[0], p[0], u[0])
    ry = supy - mconv.lcorr_valid_size(c["nfy"], c["ngy"], s[1], d[1], p[1], u[1])
    got = mconv._ext_mcorrlcorr(x, w, b, s, d, p, u, (rx, ry))
    assert tuple(got.shape) == exp.shape
    np.testing.assert_allclose(to_np(got), exp, **_tol(np.float32, c))
    if name == "mcorr1d":
        got1 = mconv._ext_mcorr1d(x[..., 0], w[..., 0], b, s[0], d[0], p[0], u[0], rx)
        np.testing.assert_allclose(to_np(got1), exp[..., 0], **_tol(np.float32, c))
