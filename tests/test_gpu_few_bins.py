"""Layers whose frequency axis has shrunk to one or two bins under a padded filter.

With 2 bins, a 4-wide filter and padding 1 the single output column has taps for filter
columns 1 and 2 only; the matrix-core plans (bf16 split, f16) leave out the filter columns
none of whose taps lies inside the signal for any output column, on correlation axes
(forward) and convolution axes (input gradient in gather form) alike.  Values must not
change: forward and both gradients against the float64 checker at rtol 1e-5 /
atol 1e-5 * sqrt(fan_in), half precision to the rounding of a half result.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu

CASES = [
    # (kind, n, c_in, c_out, nf, ng, s, d, p, r): 2 bins -> 1, filter columns 1 and 2 of 4 (the stack's last layer)
    (hip.AX_LCORR, 2, 64, 64, (4, 4), (30, 2), (1, 1), (1, 1), (1, 1), (0, 1)),
    (hip.AX_MCORR, 2, 64, 48, (4, 4), (40, 2), (1, 1), (1, 1), (1, 1), (0, 1)),
    # 1 bin, 3-wide filter: the middle column alone
    (hip.AX_LCORR, 3, 40, 33, (3, 3), (25, 1), (1, 1), (1, 1), (1, 1), (0, 1)),
    # dilation 2: columns 0 and 2 fall outside on both sides
    (hip.AX_LCORR, 2, 32, 32, (3, 3), (20, 2), (1, 1), (1, 2), (1, 2), (0, 2)),
    # stride 2 over 3 bins: every column has a tap for one of the two outputs (nothing to leave out)
    (hip.AX_LCORR, 2, 32, 40, (3, 5), (20, 3), (1, 2), (1, 1), (1, 2), (0, 1)),
    # 2 bins, padding 3 on a 4-wide filter: columns 0 and 1 only ever meet padding
    (hip.AX_MCORR, 2, 48, 32, (2, 4), (30, 2), (1, 1), (1, 1), (0, 3), (0, 0)),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_few_bins_match_checker(case, dtype):
    kind, n, c_in, c_out, nf, ng, s, d, p, r = case
    u = (1, 1)
    rng = np.random.default_rng(4100 + CASES.index(case))
    np_t = np.float32 if dtype == "float32" else np.float16
    x = rng.standard_normal((n, c_in) + ng).astype(np_t)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np_t)
    b = rng.standard_normal(c_out).astype(np_t)
    fwd = oracle.mcorrlcorr if kind == hip.AX_MCORR else oracle.lcorrlcorr
    bwd = oracle.mcorrlcorr_backward if kind == hip.AX_MCORR else oracle.lcorrlcorr_backward
    x64, w64, b64 = x.astype(np.float64), w.astype(np.float64), b.astype(np.float64)
    exp = fwd(x64, w64, b64, s, d, p, u, r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal(exp.shape).astype(np_t)
    egi, egw, _ = bwd(x64, w64, go.astype(np.float64), s, d, p, u)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
    xg, wg, bg, gog = to_gpu(x), to_gpu(w), to_gpu(b), to_gpu(go)
    tdt = torch.float32 if dtype == "float32" else torch.float16

    def close(got, e, fan, what):
        if dtype == "float32":
            assert_close(got, e, fan, what)
        else:
            err = np.abs(got.double().cpu().numpy() - e)
            assert np.all(err <= 2.0 ** -10 * np.abs(e) + 2e-5 * fan ** 0.5), what

    # (small layers stay on the fp32 instructions by default: ask for the bf16 form by name)
    hip.set_math(hip.MATH_BF16X3_ALWAYS)
    try:
        out = torch.full(exp.shape, float("nan"), dtype=tdt, device="cuda")
        hip.corr2d_forward(kind, xg, wg, bg, out, dims)
        assert hip.last_math() == (hip.MATH_BF16X3 if dtype == "float32" else hip.MATH_F16), hip.last_variant()
        close(out, exp, c_in * nf[0] * nf[1], "forward %s" % (case,))
        gi = torch.full(x.shape, float("nan"), dtype=tdt, device="cuda")
        hip.corr2d_backward_input(kind, wg, gog, gi, dims)
        close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s %s" % (hip.last_variant(), case))
        gw = torch.full(w.shape, float("nan"), dtype=tdt, device="cuda")
        hip.corr2d_backward_weight(kind, xg, gog, gw, dims)
        close(gw, egw, n * nh[0] * nh[1], "grad_weight %s %s" % (hip.last_variant(), case))
    finally:
        hip.set_math(hip.MATH_BF16X3)
