"""The two ways the matrix kernels form fp32 products (mellin_set_math).

MELLIN_MATH_BF16X3 (the default) takes every fp32 operand as the exact sum of three bf16
values and a product as the six largest of the nine bf16 cross products, formed exactly by
the bf16 matrix instructions and accumulated in fp32; MELLIN_MATH_FP32 uses the fp32 matrix
instructions.  Both must meet the operator tolerance (rtol 1e-5 / atol 1e-5 * sqrt(fan_in)
against the float64 checker), and the bf16x3 mode must not be the less accurate of the two
beyond noise: its error against the float64 checker is held to 2 x the fp32 mode's on the
benchmark's layer (all three passes of both layer kinds; measured 0.7-1.1 x for the forward
pass and the input gradient and 1.3-1.7 x for the weight gradient, whose 30 000-term sums
are rounded in a different order, both an eighth of the tolerance or less).  Every call goes
through the C ABI.
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
