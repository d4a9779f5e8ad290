"""The two ways the matrix kernels form fp32 products (mellin_set_math).

MELLIN_MATH_BF16X3 (the default) takes every fp32 operand as the exact sum of three bf16
values and a product as the six largest of the nine bf16 cross products, formed exactly by
the bf16 matrix instructions and accumulated in fp32; MELLIN_MATH_FP32 uses the fp32 matrix
instructions.  Both must meet the operator tolerance (rtol 1e-5 / atol 1e-5 * sqrt(fan_in)
against the float64 checker), and the bf16x3 mode must not be the less accurate of the two
beyond noise: its error against the float64 checker is held to 2 x the fp32 mode's on the
benchmark's layer (all three passes of both layer kinds; measured 0.7-1.1 x for the forward
pass and the input gradient and 1.3-1.7 x for the weight gradient, whose 30 000-term sums
are rounded in a different order, both an eighth of the tolerance or less).  The parts are
rounded to nearest, which bounds what the three dropped cross products can amount to by
1.01 * 2^-23 of a product; a second test feeds operands whose mantissas make the parts as
large as they can be, all of one sign so that nothing cancels, and checks every output
against that bound.  A third pins what the two modes do with infinite and NaN operands.
Every call goes through the C ABI.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

KINDS = {"mconv2d": (hip.AX_MCORR, oracle.mcorrlcorr, oracle.mcorrlcorr_backward),
         "lconv2d": (hip.AX_LCORR, oracle.lcorrlcorr, oracle.lcorrlcorr_backward)}


def _run(kind_x, math, x, w, b, go, dims):
    hip.set_math(math)
    try:
        nan = float("nan")
        out = torch.full(go.shape, nan, device="cuda")
        gi = torch.full(x.shape, nan, device="cuda")
        gw = torch.full(w.shape, nan, device="cuda")
        xg, wg, gog = to_gpu(x), to_gpu(w), to_gpu(go)
        used = []
        hip.corr2d_forward(kind_x, xg, wg, to_gpu(b), out, dims)
        used.append(hip.last_math())
        hip.corr2d_backward_input(kind_x, wg, gog, gi, dims)
        used.append(hip.last_math())
        hip.corr2d_backward_weight(kind_x, xg, gog, gw, dims)
        used.append(hip.last_math())
        return to_np(out), to_np(gi), to_np(gw), used
    finally:
        hip.set_math(hip.MATH_BF16X3)


@pytest.mark.parametrize("name", ["mconv2d", "lconv2d"])
def test_both_modes_meet_the_tolerance_and_bf16x3_is_no_less_accurate(name):
    """The benchmark's layer (3 -> 64 channels, 8 x 4 taps, 41 bins) on 4 utterances of 200 frames."""
    kind_x, fwd, bwd = KINDS[name]
    rng = np.random.default_rng(11)
    n, c_in, c_out, nf, ng = 4, 3, 64, (8, 4), (200, 41)
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    bound = (c_in * nf[0] * nf[1]) ** -0.5
    w = rng.uniform(-bound, bound, (c_out, c_in) + nf).astype(np.float32)
    b = rng.uniform(-bound, bound, c_out).astype(np.float32)
    exp = fwd(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64))
    nh = exp.shape[2:]
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, egw, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64))
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    fans = (c_in * 32, c_out * 32, n * nh[0] * nh[1])
    errs = {}
    for math in (hip.MATH_FP32, hip.MATH_BF16X3):
        out, gi, gw, used = _run(kind_x, math, x, w, b, go, dims)
        if math == hip.MATH_FP32:
            assert used == [hip.MATH_FP32] * 3, used
        else:
            assert used[0] == hip.MATH_BF16X3, used       # the forward kernel has the bf16 form for every layer kind
        for got, e, fan, what in ((out, exp, fans[0], "out"), (gi, egi, fans[1], "grad_input"),
                                  (gw, egw, fans[2], "grad_weight")):
            assert_close(got, e, fan, "%s %s math %d" % (name, what, math))
            errs[(math, what)] = float(np.sqrt(np.mean((got.astype(np.float64) - e) ** 2)))
    for what in ("out", "grad_input", "grad_weight"):
        fp32, split = errs[(hip.MATH_FP32, what)], errs[(hip.MATH_BF16X3, what)]
        assert split <= 2.0 * fp32 + 1e-12, (name, what, "rms error fp32 %.3e bf16x3 %.3e" % (fp32, split))
        print("%s %s: rms error against float64  fp32 %.3e  bf16x3 %.3e" % (name, what, fp32, split))


def test_linear_layer_runs_all_passes_in_bf16x3():
    """The benchmark's linear layer has a bf16 kernel for every pass."""
    kind_x, fwd, _ = KINDS["lconv2d"]
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 3, 64, 41)).astype(np.float32)
    w = rng.standard_normal((64, 3, 8, 4)).astype(np.float32) * 0.1
    b = np.zeros(64, np.float32)
    go = rng.standard_normal((2, 64, 57, 38)).astype(np.float32)
    dims = hip._dims(2, 3, 64, (8, 4), (64, 41), (57, 38), (1, 1), (1, 1), (0, 0), (1, 1))
    _, _, _, used = _run(kind_x, hip.MATH_BF16X3, x, w, b, go, dims)
    assert used == [hip.MATH_BF16X3] * 3, used


def test_unknown_mode_is_rejected():
    assert hip.lib.mellin_set_math(7) == 1 and "unknown mode" in hip.last_error()
    assert hip.get_math() == hip.MATH_BF16X3


@pytest.mark.parametrize("math", [hip.MATH_FP32], ids=["fp32"])
@pytest.mark.parametrize("case", [
    ("lcorrlcorr", 2, 3, 64, (8, 4), (70, 41), (1, 1), (1, 1), (0, 0)),
    ("mcorrlcorr", 3, 3, 64, (8, 4), (64, 41), (1, 1), (1, 1), (0, 0)),
    ("lcorrlcorr", 2, 5, 20, (3, 5), (23, 37), (2, 1), (1, 2), (1, 3)),
    ("mcorrlcorr", 2, 40, 33, (4, 3), (50, 29), (2, 1), (1, 1), (1, 1)),
    ("lcorrlcorr", 1, 130, 70, (3, 3), (30, 21), (1, 1), (2, 1), (2, 1)),
], ids=lambda c: "%s-%dx%d" % (c[0], c[2], c[3]))
def test_fp32_mode_keeps_every_kernel_covered(case, math):
    """The fp32 matrix kernels stay selectable; the same layers as the default-mode tests
    elsewhere, all three passes, against the float64 checker."""
    op, n, c_in, c_out, nf, ng, s, d, p = case
    kind_x = hip.AX_MCORR if op == "mcorrlcorr" else hip.AX_LCORR
    fwd = getattr(oracle, op)
    bwd = getattr(oracle, op + "_backward")
    rng = np.random.default_rng(13)
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    exp = fwd(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), s, d, p)
    nh = exp.shape[2:]
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, egw, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))
    out, gi, gw, used = _run(kind_x, math, x, w, b, go, dims)
    assert used == [math] * 3
    assert_close(out, exp, c_in * nf[0] * nf[1], "out")
    assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input")
    assert_close(gw, egw, n * nh[0] * nh[1], "grad_weight")


def _adversarial(rng, shape, scale_exp):
    """Positive fp32 values whose 24-bit mantissas maximise the mid and lo parts of the three-way
    bf16 split (all ones; a half-way case after 8 bits and again after 16; alternating runs) mixed
    with random ones, exponents spread over eight binades."""
    patterns = np.array([0x7FFFFF, 0x00FFFF, 0x008080, 0x7F8080, 0x00807F, 0x7F7F7F, 0x00C0C0, 0x40FF7F,
                         0x0080FF, 0x7FFF80, 0x3F80C0, 0x00FF80], dtype=np.uint32)
    n = int(np.prod(shape))
    mant = patterns[rng.integers(0, len(patterns), n)]
    rnd = rng.integers(0, 1 << 23, n).astype(np.uint32)
    mant = np.where(rng.random(n) < 0.25, rnd, mant)
    expo = (127 + scale_exp + rng.integers(-4, 4, n)).astype(np.uint32)
    return ((expo << 23) | mant).view(np.float32).reshape(shape)


@pytest.mark.parametrize("name", ["mconv2d", "lconv2d"])
def test_worst_case_mantissas_stay_inside_the_stated_bound(name):
    """All three passes on operands built to make the dropped cross products as large as the
    split allows, every product positive.  Each result must meet the operator tolerance against
    the float64 checker AND lie within (1.01 * 2^-23 + terms * 2^-24) * sum |w x| of it: the
    dropped products plus one fp32 rounding per accumulated term.  The bf16x3 mode must also be
    no less accurate than the fp32 instructions here (rms, factor 2)."""
    kind_x, fwd, bwd = KINDS[name]
    rng = np.random.default_rng(21)
    n, c_in, c_out, nf, ng = 2, 3, 64, (8, 4), (80, 41)
    x = _adversarial(rng, (n, c_in) + ng, 0)
    w = _adversarial(rng, (c_out, c_in) + nf, -6)
    b = np.zeros(c_out, np.float32)
    exp = fwd(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64))
    nh = exp.shape[2:]
    go = _adversarial(rng, (n, c_out) + nh, 0)
    egi, egw, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64))
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    fans = (c_in * 32, c_out * 32, n * nh[0] * nh[1])
    rms = {}
    for math in (hip.MATH_FP32, hip.MATH_BF16X3):
        out, gi, gw, used = _run(kind_x, math, x, w, b, go, dims)
        for got, e, fan, what in ((out, exp, fans[0], "out"), (gi, egi, fans[1], "grad_input"),
                                  (gw, egw, fans[2], "grad_weight")):
            assert_close(got, e, fan, "%s %s math %d" % (name, what, math))
            err = np.abs(got.astype(np.float64) - e)
            # every term is positive: sum |w x| is the exact result itself
            bound = (1.01 * 2.0 ** -23 + fan * 2.0 ** -24) * e + 2.0 ** -149
            worst = float(np.max(err / bound))
            assert worst <= 1.0, (name, what, math, "error / bound = %.3f" % worst)
            rms[(math, what)] = float(np.sqrt(np.mean((err / np.maximum(e, 1e-300)) ** 2)))
    for what in ("out", "grad_input", "grad_weight"):
        fp32, split = rms[(hip.MATH_FP32, what)], rms[(hip.MATH_BF16X3, what)]
        assert split <= 2.0 * fp32 + 2.0 ** -24, (name, what, "relative rms fp32 %.3e bf16x3 %.3e" % (fp32, split))
        print("%s %s: relative rms error against float64  fp32 %.3e  bf16x3 %.3e" % (name, what, fp32, split))


@pytest.mark.parametrize("name", ["mconv2d", "lconv2d"])
def test_infinite_and_nan_operands(name):
    """Where the bf16x3 mode differs from the reference: an infinite input value.  The fp32
    matrix instructions (and the reference's multiply-adds) carry it to +-inf in every output
    that has a tap on it; cutting it into bf16 parts forms inf - inf, so the bf16x3 mode gives
    NaN in exactly those outputs.  Outputs without a tap on it are untouched in both modes, and
    a NaN input gives NaN in its outputs under both."""
    kind_x, fwd, _ = KINDS[name]
    rng = np.random.default_rng(22)
    n, c_in, c_out, nf, ng = 2, 3, 64, (8, 4), (72, 41)
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = rng.uniform(0.01, 0.1, (c_out, c_in) + nf).astype(np.float32)      # no zero weight: inf * w is never NaN
    b = rng.standard_normal(c_out).astype(np.float32)
    x[0, 1, 11, 7] = np.inf
    x[1, 2, 23, 30] = -np.inf
    x[1, 0, 5, 20] = np.nan
    with np.errstate(invalid="ignore"):
        exp = fwd(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64))
    nh = exp.shape[2:]
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    touched = ~np.isfinite(exp)
    assert touched.any() and not touched.all()
    for math in (hip.MATH_FP32, hip.MATH_BF16X3):
        hip.set_math(math)
        try:
            out = torch.full(exp.shape, 7.0, device="cuda")
            hip.corr2d_forward(kind_x, to_gpu(x), to_gpu(w), to_gpu(b), out, dims)
            assert hip.last_math() == math
            got = to_np(out)
        finally:
            hip.set_math(hip.MATH_BF16X3)
        fan = c_in * nf[0] * nf[1]
        np.testing.assert_allclose(got[~touched], exp[~touched].astype(np.float32), rtol=1e-5, atol=1e-5 * fan ** 0.5)
        if math == hip.MATH_FP32:
            # the reference's behaviour: the same infinities and NaNs in the same places
            assert np.array_equal(np.isnan(got), np.isnan(exp))
            assert np.array_equal(got[np.isinf(exp)], exp[np.isinf(exp)].astype(np.float32))
        else:
            assert np.isnan(got[touched]).all()
