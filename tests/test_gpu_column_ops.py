"""Column ops on the GPU (snd2col / col2snd / spec2col / col2spec through the C
ABI) against the reference's own tables and the CPU checker.

The gathers move data and add at most a handful of terms in the checker's
order, so float64 results must match the tables to 1e-10 and the checker
bit for bit; float32 runs are compared with the checker bit for bit as well.
"""
import itertools

import numpy as np
import pytest
import torch

import mconv
import _mellin_hip as hip
import _fixtures as fx
from _gpu import to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-10


def _cases(*names):
    return [(n, i) for n in names for i in range(fx.num_cases(n))]


def _params(c):
    nf, ng = (c["nfx"], c["nfy"]), (c["ngx"], c["ngy"])
    s, d, p, u = ((c[k + "x"], c[k + "y"]) for k in "sdpu")
    nhx = oracle.mcorr_support_size(nf[0], ng[0], s[0], d[0], p[0], u[0])
    nhy = oracle.lcorr_support_size(nf[1], ng[1], s[1], d[1], p[1], u[1])
    return nf, ng, s, d, p, u, nhx, nhy


@pytest.mark.parametrize("name,idx", _cases("snd2col", "lin2col", "spec2col"))
def test_gather_tables(name, idx):
    """gg = spec2col(g) on the reference tables (c/tests/test_spec2col.cc:33-71)."""
    c = fx.case(name, idx)
    nf, ng, s, d, p, u, nhx, nhy = _params(c)
    flags = list(itertools.product([False, True], repeat=2))
    for batch, (tg, tgg), extra in itertools.product([1, 2], flags, [0, 10]):
        g = fx.tiled(c["G"], batch, c["c_in"], ng[0], ng[1], 0, 0, tg).reshape(-1)
        exp = np.full(batch * c["c_in"] * nf[0] * nf[1] * (nhx + extra) * nhy, -12345.0)
        oracle._col_call("spec2col", g, exp, c["c_in"], batch, nf, ng, (nhx + extra, nhy),
                         s, d, p, u, tg, tgg, "port")
        if extra == 0:
            table = fx.tiled(c["H"], batch, c["c_in"], nf[0] * nf[1], nhx * nhy, 0, 0, tgg).reshape(-1)
            np.testing.assert_allclose(exp, table, rtol=0, atol=TOL)
        gg = torch.full((exp.size,), -777.0, dtype=torch.float64, device="cuda")
        hip.col_op("spec2col", to_gpu(g), gg, c["c_in"], batch, nf, ng, (nhx + extra, nhy), s, d, p, u, tg, tgg)
        np.testing.assert_array_equal(to_np(gg), exp, err_msg="%s[%d] b=%d tg=%s tgg=%s extra=%d"
                                      % (name, idx, batch, tg, tgg, extra))


@pytest.mark.parametrize("name,idx", _cases("col2snd", "col2lin", "col2spec"))
def test_scatter_tables(name, idx):
    """g = col2spec(gg): kH holds gg and kG the expected g (c/tests/test_col2spec.cc)."""
    c = fx.case(name, idx)
    nf, ng, s, d, p, u, nhx, nhy = _params(c)
    flags = list(itertools.product([False, True], repeat=2))
    for batch, (tg, tgg) in itertools.product([1, 2], flags):
        gg = fx.tiled(c["H"], batch, c["c_in"], nf[0] * nf[1], nhx * nhy, 0, 0, tgg).reshape(-1)
        table = fx.tiled(c["G"], batch, c["c_in"], ng[0], ng[1], 0, 0, tg).reshape(-1)
        g = torch.full((table.size,), -777.0, dtype=torch.float64, device="cuda")
        hip.col_op("col2spec", to_gpu(gg), g, c["c_in"], batch, nf, ng, (nhx, nhy), s, d, p, u, tg, tgg)
        np.testing.assert_allclose(to_np(g), table, rtol=0, atol=TOL,
                                   err_msg="%s[%d] b=%d tg=%s tgg=%s" % (name, idx, batch, tg, tgg))


@pytest.mark.parametrize("name,idx", _cases("snd2col", "col2snd"))
def test_1d_entry_points(name, idx):
    c = fx.case(name, idx)
    nf, ng = c["nfx"], c["ngx"]
    s, d, p, u = c["sx"], c["dx"], c["px"], c["ux"]
    nh = oracle.mcorr_support_size(nf, ng, s, d, p, u)
    g = fx.tiled(c["G"], 2, c["c_in"], ng, 1).reshape(-1)
    gg = fx.tiled(c["H"], 2, c["c_in"], nf, nh).reshape(-1)
    if name == "snd2col":
        out = torch.full((gg.size,), -1.0, dtype=torch.float64, device="cuda")
        hip.col_op("snd2col", to_gpu(g), out, c["c_in"], 2, nf, ng, nh, s, d, p, u, False, False)
        np.testing.assert_allclose(to_np(out), gg, rtol=0, atol=TOL)
    else:
        out = torch.full((g.size,), -1.0, dtype=torch.float64, device="cuda")
        hip.col_op("col2snd", to_gpu(gg), out, c["c_in"], 2, nf, ng, nh, s, d, p, u, False, False)
        np.testing.assert_allclose(to_np(out), g, rtol=0, atol=TOL)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_public_ops_random_and_gradients(dtype):
    """mconv.spec2col / snd2col (u hidden, r extra columns) equal the checker bit for
    bit, their gradients equal col2spec / col2snd of the checker, and the
    matrix-multiply identity of the reference holds:
    mcorrlcorr(x, w) == einsum(w, spec2col(x)) (tests/test_mconv.py:632-660)."""
    rng = np.random.default_rng(11)
    for trial in range(12):
        n, c_in, c_out = (int(v) for v in rng.integers(1, 5, 3))
        nf = tuple(int(v) for v in rng.integers(1, 5, 2))
        ng = tuple(int(v) for v in rng.integers(4, 30, 2))
        s = tuple(int(v) for v in rng.integers(1, 3, 2))
        d = tuple(int(v) for v in rng.integers(1, 3, 2))
        p = tuple(int(v) for v in rng.integers(0, 3, 2))
        r = tuple(int(v) for v in rng.integers(0, 3, 2))
        x = rng.standard_normal((n, c_in) + ng).astype(dtype)
        exp = oracle.spec2col(x, nf, s, d, p, 1, r)
        if exp.size == 0:
            continue
        xt = to_gpu(x).requires_grad_(True)
        got = mconv.spec2col(xt, nf, s, d, p, r)
        assert tuple(got.shape) == exp.shape
        np.testing.assert_array_equal(to_np(got), exp, err_msg="spec2col trial %d" % trial)
        go = rng.standard_normal(exp.shape).astype(dtype)
        got.backward(to_gpu(go))
        gexp = oracle.col2spec(go, ng, s, d, p, 1)
        np.testing.assert_allclose(to_np(xt.grad), gexp, rtol=1e-6 if dtype == np.float32 else 1e-12,
                                   atol=1e-6 if dtype == np.float32 else 1e-12, err_msg="col2spec trial %d" % trial)
        # the reference's "mm" formulation against the direct kernel
        w = rng.standard_normal((c_out, c_in) + nf).astype(dtype)
        direct = mconv.mcorrlcorr(to_gpu(x), to_gpu(w), None, s, d, p, r)
        mm = torch.einsum("ocxy,ncxyhw->nohw", to_gpu(w), got.detach())
        tol = 1e-4 if dtype == np.float32 else 1e-10
        torch.testing.assert_close(mm, direct, rtol=tol, atol=tol)
        # 1-D twin
        x1 = np.ascontiguousarray(x[..., 0])
        e1 = oracle.snd2col(x1, nf[0], s[0], d[0], p[0], 1, r[0])
        x1t = to_gpu(x1).requires_grad_(True)
        g1 = mconv.snd2col(x1t, nf[0], s[0], d[0], p[0], r[0])
        np.testing.assert_array_equal(to_np(g1), e1)
        go1 = rng.standard_normal(e1.shape).astype(dtype)
        g1.backward(to_gpu(go1))
        np.testing.assert_allclose(to_np(x1t.grad), oracle.col2snd(go1, ng[0], s[0], d[0], p[0], 1),
                                   rtol=1e-6 if dtype == np.float32 else 1e-12,
                                   atol=1e-6 if dtype == np.float32 else 1e-12)


def test_transposed_input_is_used_where_it_lies():
    """The layout rule of ext/torch.cpp:75-81: a (C, N, ...) tensor viewed as (N, C, ...)."""
    rng = np.random.default_rng(3)
    base = rng.standard_normal((3, 4, 20, 9)).astype(np.float32)         # (C, N, T, F) in memory
    x = to_gpu(base).transpose(0, 1)
    got = mconv.spec2col(x, (3, 2), 1, 1, 1, 0)
    exp = oracle.spec2col(np.ascontiguousarray(np.swapaxes(base, 0, 1)), (3, 2), 1, 1, 1, 1, 0)
    np.testing.assert_array_equal(to_np(got), exp)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_adjoint_with_more_than_four_filter_columns(dtype):
    """The plane adjoint requests a filter row's loads four filter columns at a time: filters
    5-9 columns wide take two or three such blocks per row, the last one part-filled, on
    both kinds of x axis (spec: Mellin x linear; a unit x axis leaves the linear y alone)."""
    rng = np.random.default_rng(23)
    for trial, (nf, ng, s, d, p, r) in enumerate([
            ((3, 5), (40, 23), (1, 1), (1, 1), (0, 0), (0, 0)),
            ((2, 7), (31, 30), (1, 2), (1, 1), (1, 3), (0, 1)),
            ((4, 9), (25, 41), (1, 1), (2, 2), (1, 2), (2, 0)),
            ((1, 6), (1, 64), (1, 1), (1, 1), (0, 2), (0, 0)),
            ((8, 8), (64, 20), (1, 1), (1, 1), (0, 0), (0, 0))]):
        x = rng.standard_normal((9, 3) + ng).astype(dtype)               # 27 pairs: three groups of eight + three
        exp = oracle.spec2col(x, nf, s, d, p, 1, r)
        assert exp.size > 0
        xt = to_gpu(x).requires_grad_(True)
        got = mconv.spec2col(xt, nf, s, d, p, r)
        np.testing.assert_array_equal(to_np(got), exp, err_msg="spec2col trial %d" % trial)
        go = rng.standard_normal(exp.shape).astype(dtype)
        got.backward(to_gpu(go))
        gexp = oracle.col2spec(go, ng, s, d, p, 1)
        tol = 2e-6 if dtype == np.float32 else 1e-12                     # sums of up to 72 terms of unit variance
        np.testing.assert_allclose(to_np(xt.grad), gexp, rtol=tol, atol=tol * np.sqrt(nf[0] * nf[1]),
                                   err_msg="col2spec trial %d" % trial)
