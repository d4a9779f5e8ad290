"""Pins for the CPU checker that do not come from the reference's tables.

* brute force straight from the index relations (mconv.h:24-25, :65, :105-107,
  :168-171) on tiny inputs, written independently of the checker's tap helper;
* the compiled reference header (oracle/_ref, when built) on random cases with
  u > 1, d[0] != d[1], r < 0 and transposed layouts;
* size functions: 1 + the largest output index having any / only in-range taps;
* the linear axis against torch.nn.functional.conv1d / conv2d / conv_transpose2d;
* gradient identities: adjointness <fwd(x; w), y> = <x, gi> = <w, gw> in float64
  and finite differences.
"""
import itertools
from fractions import Fraction

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle

HAVE_REF = oracle.have_ref()
needs_ref = pytest.mark.skipif(not HAVE_REF, reason="oracle/_ref not built (no reference checkout)")


# --------------------------------------------------------------------------
# independent brute force
# --------------------------------------------------------------------------
def _src_index(kind, h, f, s, d, p, u):
    """Signal index as an exact rational, or None if not an integer."""
    if kind == "mcorr":
        v = Fraction((h + s) * (f + d), p + 1) - u
    elif kind == "mconv":
        v = Fraction((p + 1) * (h + s), f + d) - u
    elif kind == "lcorr":
        v = Fraction(s * h + d * f - p, u)
    else:
        v = Fraction(s * h - d * f + p, u)
    return int(v) if v.denominator == 1 else None


def brute2d(kx, ky, w, x, nh, s, d, p, u):
    c_out, c_in, nfx, nfy = w.shape
    n, _, ngx, ngy = x.shape
    out = np.zeros((n, c_out, nh[0], nh[1]), dtype=np.float64)
    for hx, hy, fx_, fy in itertools.product(range(nh[0]), range(nh[1]), range(nfx), range(nfy)):
        gx = _src_index(kx, hx, fx_, s[0], d[0], p[0], u[0])
        gy = _src_index(ky, hy, fy, s[1], d[1], p[1], u[1])
        if gx is None or gy is None or not (0 <= gx < ngx and 0 <= gy < ngy):
            continue
        out[:, :, hx, hy] += np.einsum("oc,nc->no", w[:, :, fx_, fy], x[:, :, gx, gy])
    return out


KINDS = {"mcorrlcorr": ("mcorr", "lcorr"), "mconvlconv": ("mconv", "lconv"),
         "lcorrlcorr": ("lcorr", "lcorr"), "lconvlconv": ("lconv", "lconv")}
AX = {"mcorr": oracle.AX_MCORR, "mconv": oracle.AX_MCONV,
      "lcorr": oracle.AX_LCORR, "lconv": oracle.AX_LCONV}


def _rand_params(rng):
    return (tuple(int(v) for v in rng.integers(1, 4, 2)), tuple(int(v) for v in rng.integers(1, 4, 2)),
            tuple(int(v) for v in rng.integers(0, 4, 2)), tuple(int(v) for v in rng.integers(1, 4, 2)))


@pytest.mark.parametrize("op", sorted(KINDS))
def test_brute_force_tiny(op):
    rng = np.random.default_rng(7)
    kx, ky = KINDS[op]
    for trial in range(60):
        c_out, c_in, n = (int(v) for v in rng.integers(1, 4, 3))
        nf = tuple(int(v) for v in rng.integers(1, 5, 2))
        ng = tuple(int(v) for v in rng.integers(1, 8, 2))
        nh = tuple(int(v) for v in rng.integers(1, 12, 2))
        s, d, p, u = _rand_params(rng)
        w = rng.integers(-4, 5, (c_out, c_in) + nf).astype(np.float64)
        x = rng.integers(-4, 5, (n, c_in) + ng).astype(np.float64)
        h = np.zeros((n, c_out) + nh)
        oracle.kernel2d((AX[kx], AX[ky]), w.reshape(-1), x.reshape(-1), h.reshape(-1),
                        c_out, c_in, n, nf, ng, nh, s, d, p, u)
        np.testing.assert_array_equal(h, brute2d(kx, ky, w, x, nh, s, d, p, u),
                                      err_msg="%s trial %d %s" % (op, trial, (nf, ng, nh, s, d, p, u)))


def test_dirichlet_special_case():
    """s=d=u=1, p=0: h[t] = sum_tau psi[tau] x[(t+1)(tau+1)-1] (mconv.py:1084-1086)."""
    rng = np.random.default_rng(3)
    psi, x = rng.standard_normal(5), rng.standard_normal(40)
    nh = oracle.mcorr_valid_size(5, 40)
    assert nh == 8
    exp = [sum(psi[k] * x[(t + 1) * (k + 1) - 1] for k in range(5)) for t in range(nh)]
    got = oracle.mcorr1d(x.reshape(1, 1, -1), psi.reshape(1, 1, -1))
    np.testing.assert_allclose(got.reshape(-1), exp, rtol=1e-13)


# --------------------------------------------------------------------------
# against the compiled reference header
# --------------------------------------------------------------------------
@needs_ref
@pytest.mark.parametrize("op", ["mcorrlcorr", "mconvlconv"])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_port_equals_reference_random(op, dtype):
    rng = np.random.default_rng(11)
    kx, ky = KINDS[op]
    for trial in range(150):
        c_out, c_in, n = (int(v) for v in rng.integers(1, 6, 3))
        nf = tuple(int(v) for v in rng.integers(1, 7, 2))
        ng = tuple(int(v) for v in rng.integers(1, 25, 2))
        nh = tuple(int(v) for v in rng.integers(1, 40, 2))
        s, d, p, u = _rand_params(rng)
        tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
        w = rng.standard_normal(c_out * c_in * nf[0] * nf[1]).astype(dtype)
        x = rng.standard_normal(n * c_in * ng[0] * ng[1]).astype(dtype)
        h0 = rng.standard_normal(n * c_out * nh[0] * nh[1]).astype(dtype)
        a, b = h0.copy(), h0.copy()
        args = (c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        oracle.kernel2d((AX[kx], AX[ky]), w, x, a, *args, impl="port")
        oracle.kernel2d((AX[kx], AX[ky]), w, x, b, *args, impl="ref")
        # same loop order and accumulator type -> identical bits
        np.testing.assert_array_equal(a, b, err_msg="%s trial %d %s" % (op, trial, args))


@needs_ref
@pytest.mark.parametrize("kind", ["mcorr", "mconv"])
def test_port_equals_reference_1d(kind):
    """The reference's default 1-D algorithms (MCorr1D v3, MConv1D v2) walk taps differently."""
    rng = np.random.default_rng(5)
    for trial in range(200):
        c_out, c_in, n = (int(v) for v in rng.integers(1, 5, 3))
        nf, ng, nh = int(rng.integers(1, 12)), int(rng.integers(1, 60)), int(rng.integers(1, 90))
        s, d, u = (int(v) for v in rng.integers(1, 5, 3))
        p = int(rng.integers(0, 5))
        tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
        w = rng.standard_normal(c_out * c_in * nf)
        x = rng.standard_normal(n * c_in * ng)
        a = np.zeros(n * c_out * nh)
        b = a.copy()
        args = (c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        oracle.kernel1d(AX[kind], w, x, a, *args, impl="port")
        oracle.kernel1d(AX[kind], w, x, b, *args, impl="ref")
        np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12, err_msg="%s %s" % (kind, args))


@needs_ref
def test_sizes_equal_reference():
    names = ["mconv_valid", "mconv_support", "lconv_valid", "lconv_support",
             "mcorr_valid", "mcorr_support", "lcorr_valid", "lcorr_support"]
    rng = np.random.default_rng(1)
    for _ in range(3000):
        nf, ng = int(rng.integers(1, 20)), int(rng.integers(1, 800))
        s, d, u = (int(v) for v in rng.integers(1, 6, 3))
        p = int(rng.integers(0, 6))
        for nm in names:
            fn = getattr(oracle, nm + "_size")
            assert fn(nf, ng, s, d, p, u, impl="port") == fn(nf, ng, s, d, p, u, impl="ref"), (nm, nf, ng, s, d, p, u)


@needs_ref
@pytest.mark.parametrize("dims", [1, 2])
def test_backward_identities_equal_reference(dims):
    """Role-swapped backward calls through both back ends (ext/torch.cpp:193-308)."""
    rng = np.random.default_rng(2)
    for trial in range(40):
        n, c_in, c_out = (int(v) for v in rng.integers(1, 5, 3))
        s, d, p, u = _rand_params(rng)
        if dims == 1:
            nf, ng = int(rng.integers(1, 6)), int(rng.integers(4, 30))
            r = int(rng.integers(0, 3))
            x, w = rng.standard_normal((n, c_in, ng)), rng.standard_normal((c_out, c_in, nf))
            out = oracle.mcorr1d(x, w, None, s[0], d[0], p[0], u[0], r)
            if out.size == 0:
                continue
            go = rng.standard_normal(out.shape)
            a = oracle.mcorr1d_backward(x, w, go, s[0], d[0], p[0], u[0], impl="port")
            b = oracle.mcorr1d_backward(x, w, go, s[0], d[0], p[0], u[0], impl="ref")
        else:
            nf = tuple(int(v) for v in rng.integers(1, 5, 2))
            ng = tuple(int(v) for v in rng.integers(4, 16, 2))
            r = tuple(int(v) for v in rng.integers(0, 3, 2))
            x, w = rng.standard_normal((n, c_in) + ng), rng.standard_normal((c_out, c_in) + nf)
            out = oracle.mcorrlcorr(x, w, None, s, d, p, u, r)
            if out.size == 0:
                continue
            go = rng.standard_normal(out.shape)
            a = oracle.mcorrlcorr_backward(x, w, go, s, d, p, u, impl="port")
            b = oracle.mcorrlcorr_backward(x, w, go, s, d, p, u, impl="ref")
        for va, vb in zip(a, b):
            assert va.shape == vb.shape
            np.testing.assert_allclose(va, vb, rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------
# sizes from first principles
# --------------------------------------------------------------------------
@pytest.mark.parametrize("kind", ["mcorr", "mconv", "lcorr", "lconv"])
def test_sizes_from_first_principles(kind):
    """support = 1 + max output index with any in-range tap; valid = 1 + max output index
    whose every filter tap lands at or below ng-1 (the derivations in mconv.h:432-672)."""
    rng = np.random.default_rng(9)
    valid_fn = getattr(oracle, kind + "_valid_size")
    support_fn = getattr(oracle, kind + "_support_size")
    for _ in range(300):
        nf, ng = int(rng.integers(1, 6)), int(rng.integers(1, 15))
        s, d, u = (int(v) for v in rng.integers(1, 4, 3))
        p = int(rng.integers(0, 4))
        big = 400

        def pos(h, f):  # real-valued signal position of the tap
            if kind == "mcorr":
                return Fraction((h + s) * (f + d), p + 1) - u
            if kind == "mconv":
                return Fraction((p + 1) * (h + s), f + d) - u
            if kind == "lcorr":
                return Fraction(s * h + d * f - p, u)
            return Fraction(s * h - d * f + p, u)

        sup = 0
        val = 0
        for h in range(big):
            ps = [pos(h, f) for f in range(nf)]
            if min(ps) <= ng - 1:
                sup = h + 1
            if max(ps) <= ng - 1:
                val = h + 1
        assert support_fn(nf, ng, s, d, p, u) == sup, (kind, nf, ng, s, d, p, u)
        assert valid_fn(nf, ng, s, d, p, u) == val, (kind, nf, ng, s, d, p, u)


def test_tap_map_is_mask_of_kernel():
    """Zeroing the signal wherever the tap map points leaves nothing: the map is the mask."""
    m = oracle.tap_map(oracle.AX_MCORR, 8, 512, 64, 1, 1, 0, 1)
    assert m.shape == (64, 8)
    assert (m >= 0).sum() == 512                       # 512 valid (hx, fx) pairs at this shape
    assert len(np.unique(m[m >= 0])) == 269            # only 269 of 512 input rows are read
    hx, fx_ = np.nonzero(m >= 0)
    np.testing.assert_array_equal(m[hx, fx_], (hx + 1) * (fx_ + 1) - 1)


# --------------------------------------------------------------------------
# linear axis against torch's convolutions
# --------------------------------------------------------------------------
@pytest.mark.parametrize("s,d,p,r", [((1, 1), (1, 1), (0, 0), (0, 0)), ((2, 1), (1, 2), (1, 2), (1, 2)),
                                     ((1, 2), (2, 1), (2, 1), (2, 1)), ((3, 2), (2, 3), (3, 0), (0, 3))])
def test_lcorrlcorr_is_conv2d(s, d, p, r):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((3, 4, 17, 13))
    w = rng.standard_normal((5, 4, 3, 2))
    b = rng.standard_normal(5)
    got = oracle.lcorrlcorr(x, w, b, s, d, p, 1, r)
    xt = F.pad(torch.from_numpy(x), (p[1], 40, p[0], 40))
    exp = F.conv2d(xt, torch.from_numpy(w), torch.from_numpy(b), stride=s, dilation=d)
    exp = exp[:, :, :got.shape[2], :got.shape[3]].numpy()
    assert got.shape[2] == oracle.lcorr_valid_size(3, 17, s[0], d[0], p[0]) + r[0]
    np.testing.assert_allclose(got, exp, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("s,d,p", [(1, 1, 0), (2, 1, 1), (1, 2, 3), (2, 2, 0)])
def test_mcorrlcorr_unit_mellin_axis_is_conv1d(s, d, p):
    """nfx = ngx = 1 collapses the Mellin axis (c/tests/test_mcorrlcorr.cc:45-57)."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 3, 1, 50))
    w = rng.standard_normal((4, 3, 1, 5))
    got = oracle.mcorrlcorr(x, w, None, (1, s), (1, d), (0, p), 1, 0)
    exp = F.conv1d(F.pad(torch.from_numpy(x[:, :, 0]), (p, 0)), torch.from_numpy(w[:, :, 0]),
                   stride=s, dilation=d).numpy()
    np.testing.assert_allclose(got[:, :, 0], exp, rtol=1e-12, atol=1e-12)


def test_lconvlconv_is_conv_transpose2d():
    """Linear convolution with upsampling u is a transposed convolution with stride u."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 3, 6, 7))
    w = rng.standard_normal((4, 3, 3, 2))          # (c_out, c_in, kx, ky) in the op's own layout
    for u, d in (((1, 1), (1, 1)), ((2, 3), (1, 1)), ((2, 1), (2, 3))):
        nh = tuple(oracle.lconv_support_size(w.shape[2 + i], x.shape[2 + i], 1, d[i], 0, u[i]) for i in range(2))
        h = np.zeros((2, 4) + nh)
        oracle.kernel2d((oracle.AX_LCONV, oracle.AX_LCONV), w.reshape(-1), x.reshape(-1), h.reshape(-1),
                        4, 3, 2, w.shape[2:], x.shape[2:], nh, (1, 1), d, (0, 0), u)
        exp = F.conv_transpose2d(torch.from_numpy(x), torch.from_numpy(w).transpose(0, 1),
                                 stride=u, dilation=d).numpy()
        np.testing.assert_allclose(h, exp, rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------
# gradient identities
# --------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["mcorrlcorr", "lcorrlcorr"])
def test_backward_adjointness(op):
    rng = np.random.default_rng(10)
    fwd = getattr(oracle, op)
    bwd = getattr(oracle, op + "_backward")
    checked = 0
    for trial in range(60):
        n, c_in, c_out = (int(v) for v in rng.integers(1, 4, 3))
        nf = tuple(int(v) for v in rng.integers(1, 5, 2))
        ng = tuple(int(v) for v in rng.integers(3, 14, 2))
        s, d, p, u = _rand_params(rng)
        r = tuple(int(v) for v in rng.integers(-1, 3, 2))
        x, w = rng.standard_normal((n, c_in) + ng), rng.standard_normal((c_out, c_in) + nf)
        try:
            out = fwd(x, w, None, s, d, p, u, r)
        except ValueError:
            continue  # negative output size
        if out.size == 0:
            continue
        y = rng.standard_normal(out.shape)
        gi, gw, gb = bwd(x, w, y, s, d, p, u)
        assert gi.shape == x.shape and gw.shape == w.shape
        lhs = float((out * y).sum())
        # the op is bilinear in (x, w): <fwd(x; w), y> = <x, gi> = <w, gw>
        np.testing.assert_allclose(float((x * gi).sum()), lhs, rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(float((w * gw).sum()), lhs, rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(gb, y.sum((0, 2, 3)), rtol=1e-12, atol=1e-12)
        checked += 1
    assert checked > 30


def test_backward_finite_differences():
    rng = np.random.default_rng(12)
    x, w = rng.standard_normal((2, 2, 9, 5)), rng.standard_normal((3, 2, 3, 2))
    s, d, p, u, r = (1, 2), (2, 1), (3, 1), (2, 1), (1, 1)
    out = oracle.mcorrlcorr(x, w, None, s, d, p, u, r)
    y = rng.standard_normal(out.shape)
    gi, gw, _ = oracle.mcorrlcorr_backward(x, w, y, s, d, p, u)
    eps = 1e-6
    for arr, grad in ((x, gi), (w, gw)):
        for _ in range(25):
            idx = tuple(int(rng.integers(0, k)) for k in arr.shape)
            old = arr[idx]
            arr[idx] = old + eps
            up = float((oracle.mcorrlcorr(x, w, None, s, d, p, u, r) * y).sum())
            arr[idx] = old - eps
            dn = float((oracle.mcorrlcorr(x, w, None, s, d, p, u, r) * y).sum())
            arr[idx] = old
            np.testing.assert_allclose((up - dn) / (2 * eps), grad[idx], rtol=1e-6, atol=1e-7)


def test_batching_invariance():
    """Batch N equals the batch-1 result tiled (c/tests/test_batching.cc:69-155)."""
    rng = np.random.default_rng(13)
    for c_in, c_out, nf, ng, s, d, p, u in [(1, 1, 3, 10, 1, 1, 0, 1), (16, 8, 10, 300, 2, 3, 5, 7),
                                            (4, 3, 3, 300, 1, 3, 5, 1)]:
        w = rng.uniform(-1, 1, (c_out, c_in, nf, 2)).astype(np.float32)
        x1 = rng.uniform(-1, 1, (1, c_in, ng, 6)).astype(np.float32)
        one = oracle.mcorrlcorr(x1, w, None, (s, 1), (d, 1), (p, 1), (u, 1), (2, 1))
        many = oracle.mcorrlcorr(np.repeat(x1, 5, 0), w, None, (s, 1), (d, 1), (p, 1), (u, 1), (2, 1))
        np.testing.assert_array_equal(many, np.repeat(one, 5, 0))
