"""Weight gradient: the row-wise matrix-core kernel, the tiled one and the one whose matrix
instructions run along the output positions (wide layers) must all agree with the CPU
checker through the C ABI.

Tolerance: rtol 1e-5 / atol 1e-5 * sqrt(fan_in) against the float64 checker
(fan_in = terms per output = batch * output positions).
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu

OPS = {"mcorrlcorr": (hip.AX_MCORR, oracle.mcorrlcorr, oracle.mcorrlcorr_backward),
       "lcorrlcorr": (hip.AX_LCORR, oracle.lcorrlcorr, oracle.lcorrlcorr_backward)}


def _grad_weight(kind_x, x, go, w_shape, s, d, p, u, variant):
    n, c_in, ngx, ngy = x.shape
    c_out, _, nfx, nfy = w_shape
    nhx, nhy = go.shape[2:]
    dims = hip._dims(n, c_in, c_out, (nfx, nfy), (ngx, ngy), (nhx, nhy), s, d, p, u)
    gw = torch.full(w_shape, float("nan"), dtype=torch.float32, device="cuda")   # every word must be written
    hip.set_variant(variant)
    try:
        hip.corr2d_backward_weight(kind_x, to_gpu(x), to_gpu(go), gw, dims)
        return gw, hip.last_variant()
    finally:
        hip.set_variant(None)


CASES = [
    # (op, n, c_in, c_out, nf, ng, s, d, p, u, r)
    ("lcorrlcorr", 3, 3, 64, (8, 4), (40, 41), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),   # the benchmark layer, shortened
    ("mcorrlcorr", 3, 3, 64, (8, 4), (64, 41), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),   # its Mellin twin
    ("lcorrlcorr", 2, 5, 20, (3, 5), (23, 37), (2, 1), (1, 2), (1, 3), (1, 1), (0, 0)),   # odd row length, padding, dilation
    ("mcorrlcorr", 2, 2, 33, (4, 3), (50, 29), (2, 1), (1, 1), (1, 1), (2, 1), (0, 0)),   # Mellin with s, p, u; 33 channels
    ("lcorrlcorr", 2, 7, 40, (2, 7), (11, 16), (1, 1), (2, 1), (0, 2), (1, 3), (1, 0)),   # up-sampling in y, an extra output row
    ("lcorrlcorr", 1, 40, 10, (3, 3), (19, 21), (1, 1), (1, 1), (1, 1), (1, 1), (0, 0)),  # many columns: several column blocks
    ("mcorrlcorr", 2, 1, 3, (5, 2), (30, 17), (1, 1), (2, 1), (0, 0), (1, 1), (3, 0)),    # rows past the Mellin support
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_rows_and_tiles_match_checker(case):
    op, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x, fwd, bwd = OPS[op]
    rng = np.random.default_rng(1000 + CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    nh = fwd(x, w, None, s, d, p, u, r).shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    _, exp, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    fan_in = n * nh[0] * nh[1]
    rows, v1 = _grad_weight(kind_x, x, go, w.shape, s, d, p, u, None)
    assert v1 == "mfma-rows", v1
    assert_close(rows, exp, fan_in, "rows %s" % (case,))
    tiles, v2 = _grad_weight(kind_x, x, go, w.shape, s, d, p, u, "two-pass")
    assert v2 == "mfma", v2
    assert_close(tiles, exp, fan_in, "tiles %s" % (case,))


def test_rows_is_run_to_run_deterministic():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((4, 3, 128, 41)).astype(np.float32)
    go = rng.standard_normal((4, 64, 121, 38)).astype(np.float32)
    first, v = _grad_weight(hip.AX_LCORR, x, go, (64, 3, 8, 4), (1, 1), (1, 1), (0, 0), (1, 1), None)
    assert v == "mfma-rows"
    for _ in range(3):
        again, _ = _grad_weight(hip.AX_LCORR, x, go, (64, 3, 8, 4), (1, 1), (1, 1), (0, 0), (1, 1), None)
        assert torch.equal(first, again)


WIDE_CASES = [
    # (op, n, c_in, c_out, nf, ng, s, d, p, u, r): at least 16 input and more than 32 output channels
    ("lcorrlcorr", 2, 16, 64, (3, 3), (20, 19), (1, 1), (2, 1), (2, 1), (1, 1), (0, 0)),   # dilation and padding
    ("mcorrlcorr", 3, 20, 40, (4, 2), (30, 9), (2, 1), (1, 1), (1, 0), (2, 1), (0, 0)),    # Mellin with s, p, u; 40 of 64 channel rows used
    ("lcorrlcorr", 5, 16, 200, (2, 2), (9, 5), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),    # four channel blocks side by side; rows of four outputs
    ("mcorrlcorr", 2, 41, 128, (8, 1), (100, 1), (1, 1), (1, 1), (3, 0), (1, 1), (0, 0)),  # 1-D
    ("lcorrlcorr", 2, 16, 33, (2, 3), (11, 16), (1, 2), (1, 1), (0, 2), (1, 2), (1, 0)),   # y stride and up-sampling, an extra output row
    ("lcorrlcorr", 1, 17, 70, (3, 3), (7, 6), (1, 1), (1, 1), (1, 1), (1, 1), (0, 0)),     # one image, 42 positions: a partial step only per unit
]


@pytest.mark.parametrize("case", WIDE_CASES, ids=[str(i) for i in range(len(WIDE_CASES))])
def test_positions_kernel_matches_checker(case):
    op, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x, fwd, bwd = OPS[op]
    rng = np.random.default_rng(2000 + WIDE_CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    nh = fwd(x, w, None, s, d, p, u, r).shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    _, exp, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    fan_in = n * nh[0] * nh[1]
    got, v1 = _grad_weight(kind_x, x, go, w.shape, s, d, p, u, None)
    assert v1 == "mfma-positions" and hip.last_math() == hip.MATH_BF16X3, v1
    assert_close(got, exp, fan_in, "positions %s" % (case,))
    again, _ = _grad_weight(kind_x, x, go, w.shape, s, d, p, u, None)
    assert torch.equal(got, again)                        # fixed order of summation
    other, v2 = _grad_weight(kind_x, x, go, w.shape, s, d, p, u, "two-pass")
    assert v2 == "mfma", v2
    assert_close(other, exp, fan_in, "tiles %s" % (case,))
    # no less accurate than the fp32 instructions beyond the order of summation
    err = lambda t: float(np.sqrt(np.mean((t.cpu().numpy().astype(np.float64) - exp) ** 2)))
    assert err(got) <= 3.0 * err(other) + 1e-12, (err(got), err(other))


def test_positions_kernel_needs_the_bf16_math_mode():
    """Under MELLIN_MATH_FP32 wide layers keep the fp32 kernels."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 16, 20, 19)).astype(np.float32)
    go = rng.standard_normal((2, 64, 18, 17)).astype(np.float32)
    hip.set_math(hip.MATH_FP32)
    try:
        _, v = _grad_weight(hip.AX_LCORR, x, go, (64, 16, 3, 3), (1, 1), (1, 1), (0, 0), (1, 1), None)
        assert v != "mfma-positions" and hip.last_math() == hip.MATH_FP32
    finally:
        hip.set_math(hip.MATH_BF16X3)
