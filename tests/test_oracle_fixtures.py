"""The CPU checker against every known-answer table the reference holds.

Mirrors the reference's C++ test mains: c/tests/test_mcorr1d.cc,
test_mconv1d.cc, test_mcorrlcorr.cc, test_mconvlconv.cc (which also push the
1-D Mellin and 1-D linear tables through the 2-D kernels), test_snd2col.cc,
test_col2snd.cc, test_spec2col.cc, test_col2spec.cc, over the CTest matrix of
c/tests/CMakeLists.txt:35-49 (batch, transposed_f/g/h, extra_h in {-1, 0, 10}).
float64, absolute tolerance 1e-10 as in c/tests/test_utils.h:121-150.
"""
import itertools

import numpy as np
import pytest

import _fixtures as fx
from oracle import oracle

IMPLS = ["port"] + (["ref"] if oracle.have_ref() else [])
FLAGS = list(itertools.product([False, True], repeat=3))
EXTRA = [-1, 0, 10]
TOL = 1e-10


def _cases(*names):
    return [(n, i) for n in names for i in range(fx.num_cases(n))]


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name,idx", _cases("mcorr1d", "mconv1d"))
def test_1d_tables(impl, name, idx):
    c = fx.case(name, idx)
    kind = oracle.AX_MCORR if name == "mcorr1d" else oracle.AX_MCONV
    nf, ng = c["nfx"], c["ngx"]
    s, d, p, u = c["sx"], c["dx"], c["px"], c["ux"]
    sup = (oracle.mcorr_support_size if name == "mcorr1d" else oracle.mconv_support_size)(
        nf, ng, s, d, p, u, impl=impl)
    for batch, (tf, tg, th), extra in itertools.product([1, 2], FLAGS, EXTRA):
        nh = sup + extra
        if nh <= 0:
            continue
        f = fx.filter_array(c, tf).reshape(-1)
        g = fx.tiled(c["G"], batch, c["c_in"], ng, 1, 0, 0, tg).reshape(-1)
        exp = fx.tiled(c["H"], batch, c["c_out"], sup, 1, extra, 0, th).reshape(-1)
        h = np.zeros_like(exp)
        oracle.kernel1d(kind, f, g, h, c["c_out"], c["c_in"], batch, nf, ng, nh,
                        s, d, p, u, tf, tg, th, impl=impl)
        np.testing.assert_allclose(h, exp, rtol=0, atol=TOL,
                                   err_msg="%s[%d] b=%d flags=%s extra=%d" % (name, idx, batch, (tf, tg, th), extra))


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name,idx", _cases("mcorr1d", "lcorr1d", "mcorrlcorr",
                                            "mconv1d", "lconv1d", "mconvlconv"))
def test_2d_tables(impl, name, idx):
    c = fx.case(name, idx)
    corr = name in ("mcorr1d", "lcorr1d", "mcorrlcorr")
    kinds = (oracle.AX_MCORR, oracle.AX_LCORR) if corr else (oracle.AX_MCONV, oracle.AX_LCONV)
    supx = (oracle.mcorr_support_size if corr else oracle.mconv_support_size)(
        c["nfx"], c["ngx"], c["sx"], c["dx"], c["px"], c["ux"], impl=impl)
    supy = (oracle.lcorr_support_size if corr else oracle.lconv_support_size)(
        c["nfy"], c["ngy"], c["sy"], c["dy"], c["py"], c["uy"], impl=impl)
    for batch, (tf, tg, th), extra in itertools.product([1, 2], FLAGS, EXTRA):
        nhx, nhy = supx + extra, supy + extra
        if nhx <= 0 or nhy <= 0:
            continue
        f = fx.filter_array(c, tf).reshape(-1)
        g = fx.tiled(c["G"], batch, c["c_in"], c["ngx"], c["ngy"], 0, 0, tg).reshape(-1)
        exp = fx.tiled(c["H"], batch, c["c_out"], supx, supy, extra, extra, th).reshape(-1)
        h = np.zeros_like(exp)
        oracle.kernel2d(kinds, f, g, h, c["c_out"], c["c_in"], batch,
                        (c["nfx"], c["nfy"]), (c["ngx"], c["ngy"]), (nhx, nhy),
                        (c["sx"], c["sy"]), (c["dx"], c["dy"]), (c["px"], c["py"]),
                        (c["ux"], c["uy"]), tf, tg, th, impl=impl)
        np.testing.assert_allclose(h, exp, rtol=0, atol=TOL,
                                   err_msg="%s[%d] b=%d flags=%s extra=%d" % (name, idx, batch, (tf, tg, th), extra))


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name,idx", _cases("snd2col", "lin2col", "spec2col"))
def test_gather_tables(impl, name, idx):
    """gg = spec2col(g); 1-D tables on the matching axis (c/tests/test_spec2col.cc:33-71)."""
    c = fx.case(name, idx)
    nf = (c["nfx"], c["nfy"])
    ng = (c["ngx"], c["ngy"])
    s, d, p, u = ((c[k + "x"], c[k + "y"]) for k in "sdpu")
    nhx = oracle.mcorr_support_size(nf[0], ng[0], s[0], d[0], p[0], u[0])
    nhy = oracle.lcorr_support_size(nf[1], ng[1], s[1], d[1], p[1], u[1])
    for batch, (tg, tgg), extra in itertools.product([1, 2], list(itertools.product([False, True], repeat=2)), [0, 10]):
        g = fx.tiled(c["G"], batch, c["c_in"], ng[0], ng[1], 0, 0, tg).reshape(-1)
        # the reference pads only the Mellin axis of gg (c/tests/test_spec2col.cc:76-78)
        exp = fx.tiled(c["H"], batch, c["c_in"], nf[0] * nf[1], nhx * nhy, 0, extra * nhy, tgg).reshape(-1)
        if extra:
            # rows past the support on the x axis are zero but sit inside each
            # (fx, fy) block, so rebuild the expectation block by block
            one = fx.tiled(c["H"], 1, c["c_in"], nf[0] * nf[1], nhx * nhy)[0]
            one = one.reshape(c["c_in"], nf[0] * nf[1], nhx, nhy)
            big = np.zeros((c["c_in"], nf[0] * nf[1], nhx + extra, nhy))
            big[:, :, :nhx] = one
            big = np.broadcast_to(big, (batch,) + big.shape)
            exp = np.ascontiguousarray(np.swapaxes(big, 0, 1) if tgg else big).reshape(-1)
        gg = np.full_like(exp, -12345.0)
        oracle._col_call("spec2col", g, gg, c["c_in"], batch, nf, ng, (nhx + extra, nhy),
                         s, d, p, u, tg, tgg, impl)
        np.testing.assert_allclose(gg, exp, rtol=0, atol=TOL,
                                   err_msg="%s[%d] b=%d tg=%s tgg=%s extra=%d" % (name, idx, batch, tg, tgg, extra))


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name,idx", _cases("col2snd", "col2lin", "col2spec"))
def test_scatter_tables(impl, name, idx):
    """g = col2spec(gg): kH holds gg and kG the expected g (c/tests/test_col2spec.cc)."""
    c = fx.case(name, idx)
    nf = (c["nfx"], c["nfy"])
    ng = (c["ngx"], c["ngy"])
    s, d, p, u = ((c[k + "x"], c[k + "y"]) for k in "sdpu")
    nhx = oracle.mcorr_support_size(nf[0], ng[0], s[0], d[0], p[0], u[0])
    nhy = oracle.lcorr_support_size(nf[1], ng[1], s[1], d[1], p[1], u[1])
    for batch, (tg, tgg) in itertools.product([1, 2], list(itertools.product([False, True], repeat=2))):
        gg = fx.tiled(c["H"], batch, c["c_in"], nf[0] * nf[1], nhx * nhy, 0, 0, tgg).reshape(-1)
        exp = fx.tiled(c["G"], batch, c["c_in"], ng[0], ng[1], 0, 0, tg).reshape(-1)
        g = np.full_like(exp, -12345.0)
        oracle._col_call("col2spec", gg, g, c["c_in"], batch, nf, ng, (nhx, nhy),
                         s, d, p, u, tg, tgg, impl)
        np.testing.assert_allclose(g, exp, rtol=0, atol=TOL,
                                   err_msg="%s[%d] b=%d tg=%s tgg=%s" % (name, idx, batch, tg, tgg))


@pytest.mark.parametrize("impl", IMPLS)
@pytest.mark.parametrize("name,idx", _cases("snd2col", "col2snd"))
def test_1d_column_tables(impl, name, idx):
    c = fx.case(name, idx)
    nf, ng = c["nfx"], c["ngx"]
    s, d, p, u = c["sx"], c["dx"], c["px"], c["ux"]
    nh = oracle.mcorr_support_size(nf, ng, s, d, p, u)
    g = fx.tiled(c["G"], 2, c["c_in"], ng, 1).reshape(-1)
    gg = fx.tiled(c["H"], 2, c["c_in"], nf, nh).reshape(-1)
    if name == "snd2col":
        out = np.full_like(gg, -1.0)
        oracle._col_call("snd2col", g, out, c["c_in"], 2, nf, ng, nh, s, d, p, u, False, False, impl)
        np.testing.assert_allclose(out, gg, rtol=0, atol=TOL)
    else:
        out = np.full_like(g, -1.0)
        oracle._col_call("col2snd", gg, out, c["c_in"], 2, nf, ng, nh, s, d, p, u, False, False, impl)
        np.testing.assert_allclose(out, g, rtol=0, atol=TOL)
