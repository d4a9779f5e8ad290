"""Layers whose input channels do not fit LDS at once: the kernels stage them in
chunks and keep, from a tile's first chunk (or from the same rows of the image
before), where every staged word comes from and which words are zeros.  Small
images with many channels reach those paths at a size the CPU checker does in
a blink: forward, input gradient and weight gradient through the C ABI.

Tolerance: rtol 1e-5 / atol 1e-5 * sqrt(fan_in) against the float64 checker.
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

CASES = [
    # (op, n, c_in, c_out, nf, ng, s, d, p, u, r)
    # Mellin rows of a few words (word-wise staging), 100 = 12 chunks of 8 + one of 4; 40 of 64 output channels
    ("mcorrlcorr", 6, 100, 40, (4, 4), (40, 5), (1, 1), (1, 1), (1, 1), (1, 1), (0, 0)),
    # the same with the output as long as the input (rows past the support, most virtual rows without a tap)
    ("mcorrlcorr", 2, 100, 70, (4, 4), (40, 5), (1, 1), (1, 1), (1, 1), (1, 1), (20, 0)),
    # linear rows of a few words, padding on both axes
    ("lcorrlcorr", 2, 70, 64, (4, 4), (37, 6), (1, 1), (1, 1), (1, 1), (1, 1), (0, 0)),
    # a single frequency bin left
    ("lcorrlcorr", 3, 90, 33, (4, 4), (50, 2), (1, 1), (1, 1), (1, 1), (1, 1), (0, 1)),
    # Mellin rows of 20+ words (row-wise staging) with stride, dilation and padding
    ("mcorrlcorr", 2, 150, 33, (3, 4), (60, 24), (2, 1), (1, 1), (1, 2), (1, 1), (0, 0)),
    # linear, row-wise staging, dilation and padding as in the wide benchmark layer
    ("lcorrlcorr", 2, 160, 70, (3, 3), (33, 30), (1, 1), (2, 1), (2, 1), (1, 1), (0, 0)),
    # up-sampling on both axes
    ("lcorrlcorr", 2, 120, 20, (2, 3), (20, 9), (1, 1), (1, 1), (0, 1), (2, 2), (0, 0)),
    ("mcorrlcorr", 2, 130, 20, (3, 2), (30, 7), (1, 1), (2, 1), (3, 0), (2, 1), (5, 0)),
]


def _run(kind_x, x, w, b, go, s, d, p, u):
    n, c_in, ngx, ngy = x.shape
    c_out, _, nfx, nfy = w.shape
    nhx, nhy = go.shape[2:]
    dims = hip._dims(n, c_in, c_out, (nfx, nfy), (ngx, ngy), (nhx, nhy), s, d, p, u)
    nan = float("nan")                                    # every word must be written
    out = torch.full(go.shape, nan, dtype=torch.float32, device="cuda")
    gi = torch.full(x.shape, nan, dtype=torch.float32, device="cuda")
    gw = torch.full(w.shape, nan, dtype=torch.float32, device="cuda")
    xg, wg, gog = to_gpu(x), to_gpu(w), to_gpu(go)
    hip.corr2d_forward(kind_x, xg, wg, to_gpu(b), out, dims)
    v_out = hip.last_variant()
    hip.corr2d_backward_input(kind_x, wg, gog, gi, dims)
    v_gi = hip.last_variant()
    hip.corr2d_backward_weight(kind_x, xg, gog, gw, dims)
    v_gw = hip.last_variant()
    return out, gi, gw, (v_out, v_gi, v_gw)


@pytest.fixture(params=["default", "bf16x3-always"])
def math_mode(request):
    """The default math mode leaves layers this small on the fp32 matrix instructions;
    MATH_BF16X3_ALWAYS sends them through the bf16 form of the chunked kernel as well
    (per-stage filter fragments, a short last chunk, padded taps)."""
    hip.set_math(hip.MATH_BF16X3_ALWAYS if request.param == "bf16x3-always" else hip.MATH_BF16X3)
    yield request.param
    hip.set_math(hip.MATH_BF16X3)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_chunked_layers_match_checker(case, math_mode):
    op, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x, fwd, bwd = OPS[op]
    rng = np.random.default_rng(2000 + CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    exp = fwd(x, w, b, s, d, p, u, r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, egw, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    out, gi, gw, variants = _run(kind_x, x, w, b, go, s, d, p, u)
    assert all(v.startswith("mfma") for v in variants), variants
    if math_mode == "bf16x3-always":
        hip.corr2d_forward(kind_x, to_gpu(x), to_gpu(w), to_gpu(b), torch.empty_like(out), hip._dims(
            n, c_in, c_out, nf, ng, tuple(nh), s, d, p, u))
        assert hip.last_math() == hip.MATH_BF16X3
    assert_close(out, exp, c_in * nf[0] * nf[1], "out %s" % (case,))
    assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s" % (case,))
    assert_close(gw, egw, n * nh[0] * nh[1], "grad_weight %s" % (case,))


def test_chunked_layer_is_run_to_run_deterministic():
    op, n, c_in, c_out, nf, ng, s, d, p, u, r = CASES[1]
    kind_x, fwd, _ = OPS[op]
    rng = np.random.default_rng(7)
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    b = np.zeros(c_out, np.float32)
    nh = fwd(x, w, b, s, d, p, u, r).shape[2:]
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    first = _run(kind_x, x, w, b, go, s, d, p, u)[:3]
    again = _run(kind_x, x, w, b, go, s, d, p, u)[:3]
    for a, c in zip(first, again):
        assert torch.equal(a, c)


# When a tile's staged rows are the signal's own rows the kernels copy them as one run per
# channel, 16 bytes per lane; a run of under four words has no 16-byte piece at all and is
# moved by the tail alone.  Such runs come from last tiles that hold a single short row.
SHORT_RUN_CASES = [
    # (op, n, c_in, c_out, nf, ng, s, d, p, u, r)
    # input gradient in two passes (wide Mellin layer): the first pass's last tile is one row of two words
    ("mcorrlcorr", 3, 150, 33, (5, 1), (9, 1), (1, 1), (2, 2), (0, 0), (1, 1), (0, 1)),
    # pointwise 1-D layer, 257 = 2 * 128 + 1 positions: the last tile is one word
    ("lcorrlcorr", 2, 8, 32, (1, 1), (257, 1), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),
    # rows of three words, a tile boundary that leaves one row to the last tile
    ("lcorrlcorr", 2, 20, 40, (1, 1), (43, 3), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),
    ("lcorrlcorr", 1, 3, 5, (1, 1), (3, 1), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),
]


@pytest.mark.parametrize("case", SHORT_RUN_CASES, ids=[str(i) for i in range(len(SHORT_RUN_CASES))])
def test_block_copies_of_under_four_words(case, math_mode):
    op, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x, fwd, bwd = OPS[op]
    rng = np.random.default_rng(3000 + SHORT_RUN_CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    exp = fwd(x, w, b, s, d, p, u, r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    egi, egw, _ = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)
    out, gi, gw, _ = _run(kind_x, x, w, b, go, s, d, p, u)
    assert_close(out, exp, c_in * nf[0] * nf[1], "out %s" % (case,))
    assert_close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s" % (case,))
    assert_close(gw, egw, n * nh[0] * nh[1], "grad_weight %s" % (case,))
