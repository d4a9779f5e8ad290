"""Input gradient of layers with few input channels: the fused matrix-core
kernel (linear x axis) and the two-pass path must both agree with the CPU
checker, and with each other, through the C ABI.

Tolerance: rtol 1e-5 / atol 1e-5 * sqrt(fan_in) against the float64 checker.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu


def _grad_input(kind_x, w, go, in_shape, s, d, p, u, variant):
    """grad_input of the correlation layer through mellin_corr2d_backward_input_f32."""
    n, c_in, ngx, ngy = in_shape
    c_out, _, nfx, nfy = w.shape
    nhx, nhy = go.shape[2:]
    dims = hip._dims(n, c_in, c_out, (nfx, nfy), (ngx, ngy), (nhx, nhy), s, d, p, u)
    gi = torch.full(in_shape, float("nan"), dtype=torch.float32, device="cuda")   # every word must be written
    hip.set_variant(variant)
    try:
        hip.corr2d_backward_input(kind_x, to_gpu(w), to_gpu(go), gi, dims)
        return gi, hip.last_variant()
    finally:
        hip.set_variant(None)


def _expected(x_shape, w, go, s, d, p, u):
    x = np.zeros(x_shape, dtype=np.float64)
    gi, _, _ = oracle.lcorrlcorr_backward(x, w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    return gi


CASES = [
    # (n, c_in, c_out, nf, ng, s, d, p, r)   r: output rows/cols beyond the valid size
    (2, 3, 64, (8, 4), (70, 41), (1, 1), (1, 1), (0, 0), (0, 0)),      # the benchmark layer, shortened
    (3, 1, 7, (5, 5), (33, 29), (1, 1), (1, 1), (2, 1), (0, 0)),       # one input channel, padding
    (2, 2, 33, (6, 4), (50, 20), (2, 1), (1, 2), (1, 0), (0, 0)),      # stride in x, dilation in y
    (1, 4, 100, (4, 7), (41, 37), (1, 3), (2, 1), (3, 2), (0, 0)),     # c_out past 64, stride in y, dilation in x
    (2, 3, 128, (7, 8), (64, 30), (3, 2), (2, 2), (0, 3), (0, 0)),     # two tap tiles per channel
    (2, 5, 16, (3, 9), (25, 45), (1, 1), (3, 1), (1, 1), (2, 1)),      # outputs past the valid size
    (1, 2, 5, (30, 1), (200, 1), (1, 1), (1, 1), (0, 0), (0, 0)),      # 1-D layer, long filter
    (2, 3, 64, (8, 4), (9, 6), (1, 1), (1, 1), (0, 0), (0, 0)),        # image barely larger than the filter
    (1, 1, 1, (6, 4), (300, 11), (4, 1), (1, 1), (5, 0), (0, 0)),      # stride larger than the strips' overlap
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_fused_and_two_pass_match_checker(case):
    n, c_in, c_out, nf, ng, s, d, p, r = case
    u = (1, 1)
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    nh = tuple(oracle.lcorr_valid_size(nf[i], ng[i], s[i], d[i], p[i], u[i]) + r[i] for i in range(2))
    assert min(nh) > 0
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    exp = _expected((n, c_in) + ng, w, go, s, d, p, u)
    fan_in = c_out * nf[0] * nf[1]
    fused, v1 = _grad_input(hip.AX_LCORR, w, go, (n, c_in) + ng, s, d, p, u, None)
    assert v1 == "mfma-fused", v1
    assert_close(fused, exp, fan_in, "fused %s" % (case,))
    other, v2 = _grad_input(hip.AX_LCORR, w, go, (n, c_in) + ng, s, d, p, u, "two-pass")
    assert v2 != "mfma-fused", v2
    assert_close(other, exp, fan_in, "%s %s" % (v2, case))


def test_fused_random_sweep():
    rng = np.random.default_rng(77)
    fused_seen = 0
    for trial in range(40):
        n, c_in = int(rng.integers(1, 4)), int(rng.integers(1, 6))
        c_out = int(rng.choice([1, 3, 20, 32, 40, 64, 65, 128]))
        nf = (int(rng.integers(2, 9)), int(rng.integers(2, 9)))
        ng = (int(rng.integers(nf[0], 90)), int(rng.integers(nf[1], 60)))
        s = tuple(int(v) for v in rng.integers(1, 4, 2))
        d = tuple(int(v) for v in rng.integers(1, 3, 2))
        p = tuple(int(v) for v in rng.integers(0, 4, 2))
        u = (1, 1)
        nh = tuple(oracle.lcorr_valid_size(nf[i], ng[i], s[i], d[i], p[i], u[i]) for i in range(2))
        if min(nh) <= 0:
            continue
        w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
        go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
        exp = _expected((n, c_in) + ng, w, go, s, d, p, u)
        got, v = _grad_input(hip.AX_LCORR, w, go, (n, c_in) + ng, s, d, p, u, None)
        fused_seen += v == "mfma-fused"
        assert_close(got, exp, c_out * nf[0] * nf[1], "trial %d %s nf=%s ng=%s s=%s d=%s p=%s c=%d->%d" %
                     (trial, v, nf, ng, s, d, p, c_in, c_out))
    assert fused_seen >= 10, fused_seen


def test_fused_is_run_to_run_deterministic():
    rng = np.random.default_rng(5)
    w = rng.standard_normal((64, 3, 8, 4)).astype(np.float32)
    go = rng.standard_normal((4, 64, 121, 38)).astype(np.float32)
    first, v = _grad_input(hip.AX_LCORR, w, go, (4, 3, 128, 41), (1, 1), (1, 1), (0, 0), (1, 1), None)
    assert v == "mfma-fused"
    for _ in range(3):
        again, _ = _grad_input(hip.AX_LCORR, w, go, (4, 3, 128, 41), (1, 1), (1, 1), (0, 0), (1, 1), None)
        assert torch.equal(first, again)


MELLIN_CASES = [
    # (kind, n, c_in, c_out, nf, ng, s, d, p, u, r)
    ("mcorr", 2, 3, 64, (8, 4), (96, 41), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),     # the benchmark layer, shortened
    ("mcorr", 3, 1, 7, (5, 5), (40, 29), (1, 1), (2, 1), (1, 1), (2, 1), (0, 0)),      # s, d, p, u on the Mellin axis
    ("mcorr", 2, 2, 100, (6, 4), (33, 20), (2, 2), (1, 2), (0, 3), (1, 1), (3, 1)),    # rows past the support, y stride
    ("lcorr", 2, 4, 33, (4, 7), (30, 25), (1, 1), (2, 1), (3, 2), (2, 3), (0, 0)),     # linear x with up-sampling: no fused kernel
    ("mcorr", 1, 3, 16, (7, 8), (50, 30), (1, 1), (1, 1), (2, 0), (1, 2), (0, 0)),     # two tap tiles per channel
]


@pytest.mark.parametrize("case", MELLIN_CASES, ids=[str(i) for i in range(len(MELLIN_CASES))])
def test_tap_product_and_two_pass_match_checker(case):
    kind, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x = hip.AX_MCORR if kind == "mcorr" else hip.AX_LCORR
    fwd = oracle.mcorrlcorr if kind == "mcorr" else oracle.lcorrlcorr
    bwd = oracle.mcorrlcorr_backward if kind == "mcorr" else oracle.lcorrlcorr_backward
    rng = np.random.default_rng(500 + MELLIN_CASES.index(case))
    x = np.zeros((n, c_in) + ng, dtype=np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    nh = fwd(x, w, None, s, d, p, u, r).shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    exp, _, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    fan_in = c_out * nf[0] * nf[1]
    got, v1 = _grad_input(kind_x, w, go, (n, c_in) + ng, s, d, p, u, None)
    assert v1 == "mfma-taps+fold", v1
    assert_close(got, exp, fan_in, "taps %s" % (case,))
    other, v2 = _grad_input(kind_x, w, go, (n, c_in) + ng, s, d, p, u, "two-pass")
    assert v2 != "mfma-taps+fold", v2
    assert_close(other, exp, fan_in, "%s %s" % (v2, case))


WIDE_MELLIN_CASES = [
    # (n, c_in, c_out, nf, ng, s, d, p, u): Mellin layers with many input channels whose output has
    # under 7/8 of the input's rows: dense first pass over grad_out's rows, then the fold
    (2, 20, 40, (5, 3), (60, 17), (1, 1), (1, 1), (0, 1), (1, 1)),
    (3, 41, 33, (8, 1), (100, 1), (1, 1), (2, 1), (3, 0), (1, 1)),                  # 1-D, as BASELINE config 2
    (2, 16, 64, (3, 3), (50, 12), (2, 1), (1, 2), (1, 0), (2, 1)),
]


@pytest.mark.parametrize("case", WIDE_MELLIN_CASES, ids=[str(i) for i in range(len(WIDE_MELLIN_CASES))])
def test_wide_mellin_layers_take_the_dense_two_pass_path(case):
    n, c_in, c_out, nf, ng, s, d, p, u = case
    rng = np.random.default_rng(900 + WIDE_MELLIN_CASES.index(case))
    x = np.zeros((n, c_in) + ng, dtype=np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    nh = oracle.mcorrlcorr(x, w, None, s, d, p, u, 0).shape[2:]
    assert min(nh) > 0 and 8 * nh[0] <= 7 * ng[0]
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    exp, _, _ = oracle.mcorrlcorr_backward(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64),
                                           s, d, p, u)
    got, v = _grad_input(hip.AX_MCORR, w, go, (n, c_in) + ng, s, d, p, u, None)
    assert v == "mfma+fold", v
    assert_close(got, exp, c_out * nf[0] * nf[1], "two-pass %s" % (case,))
    other, v2 = _grad_input(hip.AX_MCORR, w, go, (n, c_in) + ng, s, d, p, u, "generic")
    assert v2 == "generic", v2
    assert_close(other, exp, c_out * nf[0] * nf[1], "generic %s" % (case,))


# Tap products with the four filter columns of a filter row summed in the kernel (Y, a quarter
# of the tap products, goes through the workspace; a fold over x finishes): rows of exactly 64
# positions per image pair (the last row's tail then takes a chunk of its own), left padding,
# outputs past the valid size (grad_input narrower than the taps reach), the shortest rows the
# form takes (three positions), and rows too short for it (the per-column form runs).
YFOLD_CASES = [
    # (kind, n, c_in, c_out, nf, ng, s, d, p, r, summed in the kernel)
    (hip.AX_MCORR, 2, 3, 64, (8, 4), (64, 19), (1, 1), (1, 1), (0, 0), (0, 0), True),
    (hip.AX_MCORR, 3, 2, 33, (3, 4), (30, 6), (1, 1), (1, 1), (1, 3), (0, 0), True),
    (hip.AX_MCORR, 1, 5, 16, (5, 4), (40, 5), (1, 1), (1, 1), (0, 1), (0, 1), True),
    (hip.AX_MCORR, 2, 1, 8, (2, 4), (21, 6), (1, 1), (1, 1), (0, 0), (0, 0), True),
    (hip.AX_MCORR, 2, 3, 16, (2, 4), (20, 5), (1, 1), (1, 1), (0, 0), (0, 0), False),
    (hip.AX_MCORR, 2, 3, 16, (2, 4), (20, 9), (1, 2), (1, 1), (0, 0), (0, 0), False),   # stride along y
]


@pytest.mark.parametrize("case", YFOLD_CASES, ids=[str(i) for i in range(len(YFOLD_CASES))])
def test_tap_products_summed_over_filter_columns(case):
    import mconv
    kind, n, c_in, c_out, nf, ng, s, d, p, r, summed = case
    u = (1, 1)
    valid_x = mconv.mcorr_valid_size if kind == hip.AX_MCORR else mconv.lcorr_valid_size
    nh = (valid_x(nf[0], ng[0], s[0], d[0], p[0], 1) + r[0], mconv.lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], 1) + r[1])
    assert min(nh) > 0
    rng = np.random.default_rng(5100 + YFOLD_CASES.index(case))
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    bwd = oracle.mcorrlcorr_backward if kind == hip.AX_MCORR else oracle.lcorrlcorr_backward
    exp, _, _ = bwd(np.zeros((n, c_in) + ng), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
    need = hip.lib.mellin_corr2d_backward_input_workspace(kind, 4, *dims)
    assert need == 4 * n * c_in * (nf[0] * nh[0] * ng[1] if summed else 32 * nh[0] * nh[1])
    got, v = _grad_input(kind, w, go, (n, c_in) + ng, s, d, p, u, None)
    assert v == "mfma-taps+fold", v
    assert_close(got, exp, c_out * nf[0] * nf[1], "filter columns summed %s" % (case,))
    other, v = _grad_input(kind, w, go, (n, c_in) + ng, s, d, p, u, "tap-columns")
    assert v == "mfma-taps+fold", v
    assert_close(other, exp, c_out * nf[0] * nf[1], "per column %s" % (case,))
