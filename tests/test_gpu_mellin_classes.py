"""A Mellin layer as one launch of the tiled kernel per residue class of its x axis.

On a Mellin correlation axis the tap of (output row h, filter row f) exists iff
(h + s)(f + d) is a multiple of p + 1, so the rows with the same (h + s) mod (p + 1) have
taps for the same filter rows; on a convolution axis (the input gradient in gather form)
rows with the same (h + s) mod lcm_f((f + d) / gcd(f + d, p + 1)) do.  A launch over one
class walks only the filter rows that class has and writes only its rows: the union of
the launches must be the layer, to the operator tolerance against the float64 checker
(rtol 1e-5 / atol 1e-5 * sqrt(fan_in)) in fp32 and to the rounding of a half result
against the single launch in half precision.  The "classes" variant forces the form on
layers of any size; by default forward passes of 4 GMAC (taps without a source counted)
and more take it.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu

CASES = [
    # (n, c_in, c_out, nf, ng, s, d, p, r): two classes, the stack's layer shape, rows past the support
    (2, 100, 70, (4, 4), (40, 5), (1, 1), (1, 1), (1, 1), (20, 0)),
    # four classes, two of them with one filter row of four; row-wise staging
    (2, 40, 33, (4, 3), (60, 24), (1, 1), (1, 1), (3, 2), (7, 0)),
    # three classes, stride and dilation: class r has the filter rows with r (f + 2) a multiple of 3
    (3, 20, 64, (6, 2), (50, 9), (2, 1), (2, 1), (2, 0), (0, 1)),
    # few channels (one chunk), eight filter rows, 1-D
    (4, 3, 40, (8, 1), (90, 1), (1, 1), (1, 1), (3, 0), (10, 0)),
    # a class without output rows (one output row, two classes)
    (2, 16, 16, (2, 2), (2, 8), (1, 1), (1, 1), (1, 0), (0, 0)),
]


seen_gi = []


@pytest.fixture
def classes_forced():
    hip.set_variant("classes")
    yield
    hip.set_variant(None)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_classes_match_checker(case, classes_forced):
    n, c_in, c_out, nf, ng, s, d, p, r = case
    rng = np.random.default_rng(3000 + CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    exp = oracle.mcorrlcorr(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), s, d, p, (1, 1), r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, _, _ = oracle.mcorrlcorr_backward(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64),
                                           s, d, p, (1, 1))
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))
    out = torch.full(exp.shape, float("nan"), device="cuda")                 # every word must be written
    hip.corr2d_forward(hip.AX_MCORR, to_gpu(x), to_gpu(w), to_gpu(b), out, dims)
    single_row = nh[0] == 1
    assert hip.last_variant() == ("mfma" if single_row else "mfma-classes")  # one class with rows: nothing to split
    assert_close(out, exp, c_in * nf[0] * nf[1], "forward %s" % (case,))
    if c_in >= 16 and not single_row:
        # the gather-form input gradient is a convolution axis
        gi = torch.full(x.shape, float("nan"), device="cuda")
        hip.corr2d_backward_input(hip.AX_MCORR, to_gpu(w), to_gpu(go), gi, dims)
        seen_gi.append(hip.last_variant())                                   # (layers that keep fewer rows than they are given take two passes)
        assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s" % (case,))


def test_half_classes_match_the_single_launch(classes_forced):
    for case in CASES[:3]:
        n, c_in, c_out, nf, ng, s, d, p, r = case
        gen = torch.Generator().manual_seed(9)
        x = torch.randn((n, c_in) + ng, generator=gen).half().cuda()
        w = (torch.randn((c_out, c_in) + nf, generator=gen) * (c_in * nf[0] * nf[1]) ** -0.5).half().cuda()
        b = torch.randn(c_out, generator=gen).half().cuda()
        import mconv
        nh = (mconv.mcorr_valid_size(nf[0], ng[0], s[0], d[0], p[0], 1) + r[0],
              mconv.lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], 1) + r[1])
        dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))
        got = torch.full((n, c_out) + nh, float("nan"), dtype=torch.float16, device="cuda")
        hip.corr2d_forward(hip.AX_MCORR, x, w, b, got, dims)
        # (classes that are all staged in chunks of channels share one launch: the first layer's)
        assert hip.last_variant() == ("mfma-f16-classes" if case is CASES[0] else "mfma-f16-class-launches"), case
        hip.set_variant("class-launches")
        each = torch.full_like(got, float("nan"))
        hip.corr2d_forward(hip.AX_MCORR, x, w, b, each, dims)
        assert hip.last_variant() == "mfma-f16-class-launches" and torch.equal(each, got)   # the same plans, the same sums
        hip.set_variant("one-launch")
        ref = torch.full_like(got, float("nan"))
        hip.corr2d_forward(hip.AX_MCORR, x, w, b, ref, dims)
        assert hip.last_variant() == "mfma-f16"
        hip.set_variant("classes")
        tol = 2.0 ** -10 * ref.float().abs() + 2e-5 * (c_in * nf[0] * nf[1]) ** 0.5
        assert bool(((got.float() - ref.float()).abs() <= tol).all()), case


def test_large_forward_passes_take_the_classes_by_default():
    """5 GMAC with the taps without a source counted: one launch per class, and the same
    values as the single launch up to the order of summation."""
    n, c_in, c_out, nf, ng, p = 8, 128, 128, (4, 4), (120, 20), (1, 1)
    gen = torch.Generator().manual_seed(10)
    x = torch.randn((n, c_in) + ng, generator=gen).cuda()
    w = (torch.randn((c_out, c_in) + nf, generator=gen) * (c_in * 16) ** -0.5).cuda()
    b = torch.randn(c_out, generator=gen).cuda()
    import mconv
    nh = (mconv.mcorr_valid_size(4, 120, 1, 1, 1, 1) + 60, mconv.lcorr_valid_size(4, 20, 1, 1, 1, 1) + 2)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), p, (1, 1))
    got = torch.full((n, c_out) + nh, float("nan"), device="cuda")
    hip.corr2d_forward(hip.AX_MCORR, x, w, b, got, dims)
    assert hip.last_variant() == "mfma-classes" and hip.last_math() == hip.MATH_BF16X3
    hip.set_variant("one-launch")
    try:
        ref = torch.full_like(got, float("nan"))
        hip.corr2d_forward(hip.AX_MCORR, x, w, b, ref, dims)
        assert hip.last_variant() == "mfma"
    finally:
        hip.set_variant(None)
    assert bool(((got - ref).abs() <= 1e-5 * ref.abs() + 1e-5 * (c_in * 16) ** 0.5).all())
    # (this layer keeps its 120 rows while the taps of filter rows 2 and 3 end at rows 79 and 59:
    # by default a class's rows are cut there and all ranges share a launch; uncut, a launch per
    # class -- the same products in the same order, the rows of zeros left out or not)
    hip.set_variant("whole-classes")
    try:
        whole = torch.full_like(got, float("nan"))
        hip.corr2d_forward(hip.AX_MCORR, x, w, b, whole, dims)
        assert hip.last_variant() == "mfma-classes"
    finally:
        hip.set_variant(None)
    assert torch.equal(whole, got)


# Input gradients in two passes (layers that keep fewer rows than they are given): the first
# pass as a launch per filter row, each over the rows of grad_out that have a tap of it.
ROW_CASES = [
    # (n, c_in, c_out, nf, ng, s, d, p, r): steps 3, 1, 3 (the wide benchmark layer in small)
    (2, 64, 40, (3, 3), (60, 9), (1, 1), (2, 1), (2, 1), (0, 0)),
    # steps 2, 1, 2, 1 and rows past the support (taps beyond grad_input)
    (2, 128, 32, (4, 4), (80, 5), (1, 1), (1, 1), (1, 1), (5, 0)),
    # p + 1 = 4: steps 4, 2, 4, 1, 4, 2; stride 2
    (1, 96, 33, (6, 2), (90, 7), (2, 1), (1, 1), (3, 0), (0, 0)),
    # p + 1 = 6: steps 6, 3, 2, 3, 6, 1, 6, 3
    (2, 64, 16, (8, 1), (120, 6), (1, 1), (1, 1), (5, 0), (0, 0)),
    # 1-D, dilation 3 with p + 1 = 3: steps 1, 3, 3, 1
    (3, 64, 20, (4, 1), (100, 1), (1, 1), (3, 1), (2, 0), (0, 0)),
    # layers that keep their rows, as in the 10-layer stack: the form from 256 products per
    # first-pass word on (c_out * nfy), in half precision from 512 on
    (2, 64, 64, (4, 4), (40, 6), (1, 1), (1, 1), (1, 1), (20, 0)),
    (1, 32, 256, (4, 4), (40, 6), (1, 1), (1, 1), (1, 1), (20, 0)),
    # one output column under a dilated 8-wide filter: the first pass keeps filter columns 1-4
    # only, and the filter row's offset into the weight is still counted in whole filter rows
    (2, 64, 130, (4, 8), (35, 8), (1, 1), (1, 2), (1, 2), (3, 1)),
]


def _row_case(case, seed):
    import mconv
    n, c_in, c_out, nf, ng, s, d, p, r = case
    nh = (mconv.mcorr_valid_size(nf[0], ng[0], s[0], d[0], p[0], 1) + r[0],
          mconv.lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], 1) + r[1])
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_out * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    return nh, w, go, hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))


@pytest.mark.parametrize("case", ROW_CASES, ids=[str(i) for i in range(len(ROW_CASES))])
def test_first_pass_per_filter_row_matches_checker(case, classes_forced):
    n, c_in, c_out, nf, ng, s, d, p, r = case
    nh, w, go, dims = _row_case(case, 3100 + ROW_CASES.index(case))
    x0 = np.zeros((n, c_in) + ng)
    egi, _, _ = oracle.mcorrlcorr_backward(x0, w.astype(np.float64), go.astype(np.float64), s, d, p, (1, 1))
    gi = torch.full((n, c_in) + ng, float("nan"), device="cuda")
    hip.corr2d_backward_input(hip.AX_MCORR, to_gpu(w), to_gpu(go), gi, dims)
    assert hip.last_variant() == "mfma-filter-rows+fold" and hip.last_math() == hip.MATH_BF16X3
    assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s" % (case,))
    # the single launch sums the same products in the same order
    hip.set_variant("one-launch")
    try:
        ref = torch.full_like(gi, float("nan"))
        hip.corr2d_backward_input(hip.AX_MCORR, to_gpu(w), to_gpu(go), ref, dims)
        assert hip.last_variant() == ("mfma+fold" if 8 * nh[0] <= 7 * ng[0] else "mfma")
    finally:
        hip.set_variant("classes")
    if hip.last_math() == hip.MATH_BF16X3 and hip.last_variant() == "mfma+fold":
        assert torch.equal(gi, ref)


@pytest.mark.parametrize("case", ROW_CASES, ids=[str(i) for i in range(len(ROW_CASES))])
def test_half_first_pass_per_filter_row(case, classes_forced):
    n, c_in, c_out, nf, ng, s, d, p, r = case
    nh, w, go, dims = _row_case(case, 3200 + ROW_CASES.index(case))
    wh, goh = torch.from_numpy(w).half().cuda(), torch.from_numpy(go).half().cuda()
    gi = torch.full((n, c_in) + ng, float("nan"), dtype=torch.float16, device="cuda")
    hip.corr2d_backward_input(hip.AX_MCORR, wh, goh, gi, dims)
    if 8 * nh[0] > 7 * ng[0] and c_out * nf[1] < 512:
        assert hip.last_variant() in ("mfma-f16-classes", "mfma-f16-class-launches")   # the gather form
        return
    assert hip.last_variant() == "mfma-f16-filter-rows+fold"
    hip.set_variant("one-launch")
    try:
        ref = torch.full_like(gi, float("nan"))
        hip.corr2d_backward_input(hip.AX_MCORR, wh, goh, ref, dims)
        single = hip.last_variant()
        assert single == ("mfma-f16+fold" if 8 * nh[0] <= 7 * ng[0] else "mfma-f16")
    finally:
        hip.set_variant("classes")
    if single == "mfma-f16+fold":
        assert torch.equal(gi, ref)                                           # the same sums, rounded once
    egi, _, _ = oracle.mcorrlcorr_backward(np.zeros((n, c_in) + ng), wh.cpu().double().numpy(),
                                           goh.cpu().double().numpy(), s, d, p, (1, 1))
    err = (gi.double().cpu().numpy() - egi)
    assert np.all(np.abs(err) <= 2.0 ** -10 * np.abs(egi) + 2e-5 * (c_out * nf[0] * nf[1]) ** 0.5)


def test_large_input_gradients_take_the_filter_rows_by_default():
    """A first pass of 20 GMAC on a layer that keeps its rows: a launch per filter row, and the
    same values as the gather form up to the order of summation."""
    n, c_in, c_out, nf, ng, p = 16, 128, 256, (4, 4), (120, 20), (1, 1)
    import mconv
    nh = (mconv.mcorr_valid_size(4, 120, 1, 1, 1, 1) + 60, mconv.lcorr_valid_size(4, 20, 1, 1, 1, 1) + 2)
    assert nh[0] == ng[0]
    gen = torch.Generator().manual_seed(11)
    w = (torch.randn((c_out, c_in) + nf, generator=gen) * (c_out * 16) ** -0.5).cuda()
    go = torch.randn((n, c_out) + nh, generator=gen).cuda()
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), p, (1, 1))
    got = torch.full((n, c_in) + ng, float("nan"), device="cuda")
    hip.corr2d_backward_input(hip.AX_MCORR, w, go, got, dims)
    assert hip.last_variant() == "mfma-filter-rows+fold" and hip.last_math() == hip.MATH_BF16X3
    hip.set_variant("one-launch")
    try:
        ref = torch.full_like(got, float("nan"))
        hip.corr2d_backward_input(hip.AX_MCORR, w, go, ref, dims)
        assert hip.last_variant() == "mfma"
    finally:
        hip.set_variant(None)
    assert bool(((got - ref).abs() <= 1e-5 * ref.abs() + 1e-5 * (c_out * 16) ** 0.5).all())
    # half precision, from 512 products per first-pass word on: 1024 here
    gh = torch.full((n, c_in) + ng, float("nan"), dtype=torch.float16, device="cuda")
    hip.corr2d_backward_input(hip.AX_MCORR, w.half(), go.half(), gh, dims)
    assert hip.last_variant() == "mfma-f16-filter-rows+fold"
    ref16 = torch.full_like(gh, float("nan"))
    hip.set_variant("one-launch")
    try:
        hip.corr2d_backward_input(hip.AX_MCORR, w.half(), go.half(), ref16, dims)
        assert hip.last_variant() == "mfma-f16"
    finally:
        hip.set_variant(None)
    tol = 2.0 ** -10 * ref16.float().abs() + 2e-5 * (c_out * 16) ** 0.5
    assert bool(((gh.float() - ref16.float()).abs() <= tol).all())


def test_some_input_gradient_took_the_classes():
    """(after the parametrized cases of this file: tests run in the order they are written)"""
    assert "mfma-classes" in seen_gi, seen_gi


# Up-sampling on the Mellin axis (u > 1) together with strides and dilations above one: the
# residue classes, where a class's rows are cut (h_f = floor((ng - 1 + u)(p + 1) / (f + d)) - s)
# and the rows of a filter row's first pass all carry u.
U_CASES = [
    # (n, c_in, c_out, nf, ng, s, d, p, u, r)
    (2, 40, 48, (4, 3), (50, 9), (2, 1), (2, 1), (2, 1), (2, 1), (6, 0)),      # u = 2, s = d = 2, three classes
    (2, 64, 40, (5, 2), (40, 7), (3, 1), (1, 1), (3, 0), (3, 1), (0, 1)),      # u = 3, s = 3, four classes
    (1, 32, 33, (6, 2), (45, 5), (2, 1), (3, 1), (1, 0), (3, 2), (4, 0)),      # u = (3, 2), d = 3, two classes
    # rows far past the support of the later filter rows: the classes are cut into ranges
    (2, 32, 64, (4, 4), (60, 6), (1, 1), (1, 1), (1, 1), (2, 1), (50, 0)),
    (2, 48, 64, (4, 2), (70, 8), (2, 1), (2, 1), (1, 0), (3, 1), (40, 0)),
]

seen_u = []


@pytest.mark.parametrize("case", U_CASES, ids=[str(i) for i in range(len(U_CASES))])
def test_classes_with_upsampling_match_checker(case, classes_forced):
    n, c_in, c_out, nf, ng, s, d, p, u, r = case
    rng = np.random.default_rng(3300 + U_CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    exp = oracle.mcorrlcorr(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), s, d, p, u, r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, egw, _ = oracle.mcorrlcorr_backward(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64),
                                             s, d, p, u)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
    out = torch.full(exp.shape, float("nan"), device="cuda")                 # every word must be written
    hip.corr2d_forward(hip.AX_MCORR, to_gpu(x), to_gpu(w), to_gpu(b), out, dims)
    assert hip.last_variant() == "mfma-classes", case
    assert_close(out, exp, c_in * nf[0] * nf[1], "forward %s" % (case,))
    gi = torch.full(x.shape, float("nan"), device="cuda")
    hip.corr2d_backward_input(hip.AX_MCORR, to_gpu(w), to_gpu(go), gi, dims)
    seen_u.append(hip.last_variant())
    assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input [%s] %s" % (hip.last_variant(), case))
    gw = torch.full(w.shape, float("nan"), device="cuda")
    hip.corr2d_backward_weight(hip.AX_MCORR, to_gpu(x), to_gpu(go), gw, dims)
    assert_close(gw, egw, n * nh[0] * nh[1], "grad_weight [%s] %s" % (hip.last_variant(), case))


def test_some_upsampled_input_gradient_took_the_filter_rows():
    assert "mfma-filter-rows+fold" in seen_u, seen_u
