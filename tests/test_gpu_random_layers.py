"""Seeded random sweeps of whole layers through the C ABI against the CPU checker.

The committed parity tests pin chosen shapes; the kernels' dispatch, however, has many forms
(tiled, per residue class, fused and tap-product input gradients, row-wise / position-wise weight
gradients, filter columns left out of the plan, half precision, accumulate-into-h) whose
thresholds depend on every size at once.  Each sweep here draws layers of one family at random
(both layer kinds, strides, dilations, paddings, up-sampling, extra output rows), runs forward,
input gradient and weight gradient on the GPU with NaN-prefilled results, and compares with the
checker in float64 on the same operands at the operator tolerance (rtol 1e-5, atol
1e-5 * sqrt(fan_in); half precision: the result's rounding to half on top, rtol 1e-3).  A sweep
stops at its first mismatch, at `COUNT` layers, or after `SECONDS` of wall-clock, whichever comes
first, and must have covered at least `MIN_COUNT` layers; sizes are kept small enough for the CPU
side to take some ten milliseconds per layer.  The seeds are fixed: a failure names a reproducible
layer.
"""
import time

import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

COUNT, MIN_COUNT, SECONDS = 300, 60, 9.0

OPS = {"mcorrlcorr": (hip.AX_MCORR, oracle.mcorrlcorr, oracle.mcorrlcorr_backward),
       "lcorrlcorr": (hip.AX_LCORR, oracle.lcorrlcorr, oracle.lcorrlcorr_backward)}


def _draw(rng, family):
    """One layer: (op, n, c_in, c_out, nf, ng, s, d, p, u, r)."""
    if family == "narrow-class":
        # linear x linear, no padding or up-sampling, unit y stride and dilation, an even number of
        # filter columns, at most 128 taps in all
        c_in = int(rng.integers(1, 17))
        nfy = int(rng.choice([2, 4, 6]))
        nfx = int(rng.integers(1, max(2, min(9, 128 // (c_in * nfy) + 1))))
        if c_in * nfx * nfy > 128:
            nfx = 1
        c_out = int(rng.choice([1, 5, 32, 33, 64, 70, 130]))
        ng = (int(rng.integers(8, 120)), int(rng.choice([6, 7, 13, 20, 33, 41, 64])))
        return ("lcorrlcorr", int(rng.integers(1, 5)), c_in, c_out, (nfx, nfy), ng,
                (int(rng.integers(1, 4)), 1), (int(rng.integers(1, 4)), 1), (0, 0), (1, 1), (0, 0))
    op = ["mcorrlcorr", "lcorrlcorr"][int(rng.integers(2))]
    n = int(rng.integers(1, 7))
    if family == "few-channels":
        c_in = int(rng.integers(1, 9))
        c_out = int(rng.choice([1, 5, 16, 32, 33, 64, 70]))
    elif family == "wide":
        c_in = int(rng.choice([16, 17, 40, 64, 100, 130]))
        c_out = int(rng.choice([33, 40, 64, 70, 130]))
    else:
        c_in = int(rng.choice([1, 3, 8, 17, 40, 64]))
        c_out = int(rng.choice([3, 16, 32, 33, 64, 70]))
    nf = (int(rng.integers(1, 9)), int(rng.integers(1, 6)))
    if family == "few-bins":
        ng = (int(rng.integers(4, 300)), int(rng.integers(1, 7)))
        nf = (int(rng.integers(1, 6)), int(rng.integers(1, 5)))
    else:
        ng = (int(rng.integers(4, 220)), int(rng.choice([1, 2, 3, 5, 8, 13, 20, 33, 41, 45])))
    s = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    d = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    p = (int(rng.integers(0, 4)), int(rng.integers(0, 3)))
    u = (int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2])))
    r = (int(rng.choice([0, 0, 3, 10])), int(rng.choice([0, 0, 1])))
    return op, n, c_in, c_out, nf, ng, s, d, p, u, r


def _too_big(n, c_in, c_out, nf, nh):
    return n * c_out * nh[0] * nh[1] * c_in * nf[0] * nf[1] > 2.5e8 or n * c_out * nh[0] * nh[1] > 1.5e6


def _sweep(seed, family, dtype=np.float32, math=None, variant=None):
    rng = np.random.default_rng(seed)
    half = dtype == np.float16
    rtol = 1e-3 if half else 1e-5
    variants = {}
    done = 0
    if math is not None:
        hip.set_math(math)
    hip.set_variant(variant)
    t0 = time.time()
    try:
        while done < COUNT and time.time() - t0 < SECONDS:
            op, n, c_in, c_out, nf, ng, s, d, p, u, r = _draw(rng, family)
            kind_x, fwd, bwd = OPS[op]
            x = rng.standard_normal((n, c_in) + ng).astype(dtype)
            w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(dtype)
            b = rng.standard_normal(c_out).astype(dtype)
            x64, w64, b64 = x.astype(np.float64), w.astype(np.float64), b.astype(np.float64)
            try:
                exp = fwd(x64, w64, b64, s, d, p, u, r)
            except Exception:
                continue                                  # (an output extent below one)
            nh = exp.shape[2:]
            if min(nh) <= 0 or _too_big(n, c_in, c_out, nf, nh):
                continue
            go = rng.standard_normal((n, c_out) + nh).astype(dtype)
            egi, egw, _ = bwd(x64, w64, go.astype(np.float64), s, d, p, u)
            dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
            tdt = torch.float16 if half else torch.float32
            nan = float("nan")
            out = torch.full(exp.shape, nan, device="cuda", dtype=tdt)
            gi = torch.full(x.shape, nan, device="cuda", dtype=tdt)
            gw = torch.full(w.shape, nan, device="cuda", dtype=tdt)
            xg, wg, gog = to_gpu(x), to_gpu(w), to_gpu(go)
            layer = (op, n, c_in, c_out, nf, ng, s, d, p, u, r)
            hip.corr2d_forward(kind_x, xg, wg, to_gpu(b), out, dims)
            names = [hip.last_variant()]
            hip.corr2d_backward_input(kind_x, wg, gog, gi, dims)
            names.append(hip.last_variant())
            hip.corr2d_backward_weight(kind_x, xg, gog, gw, dims)
            names.append(hip.last_variant())
            for got, e, fan, what, name in ((out, exp, c_in * nf[0] * nf[1], "forward", names[0]),
                                            (gi, egi, c_out * nf[0] * nf[1], "grad_input", names[1]),
                                            (gw, egw, n * nh[0] * nh[1], "grad_weight", names[2])):
                g = to_np(got.float()).astype(np.float64)
                err = np.abs(g - e)
                tol = rtol * np.abs(e) + 1e-5 * fan ** 0.5
                assert np.all(err <= tol), "%s [%s] of layer %d %s (seed %d, family %s): worst error %.3e%s" % (
                    what, name, done, layer, seed, family, np.nanmax(err), ", NaN in the result" if np.isnan(g).any() else "")
                variants[name] = variants.get(name, 0) + 1
            done += 1
    finally:
        hip.set_variant(None)
        hip.set_math(hip.MATH_BF16X3)
    print("%s: %d layers in %.1f s, kernels %s" % (family, done, time.time() - t0, variants))
    assert done >= MIN_COUNT, "only %d layers in %.0f s" % (done, SECONDS)
    return variants


def test_default_math():
    v = _sweep(101, "any")
    assert "mfma" in v


def test_bf16x3_for_small_layers_too():
    _sweep(102, "any", math=hip.MATH_BF16X3_ALWAYS)


def test_fp32_math():
    _sweep(103, "any", math=hip.MATH_FP32)


def test_few_input_channels():
    """1-8 input channels: the fused and tap-product input gradients, the row-wise weight gradients."""
    v = _sweep(104, "few-channels")
    assert any(k in v for k in ("mfma-fused", "mfma-taps+fold"))


def test_few_frequency_bins():
    """1-6 bins: filter columns without a tap are left out of the plans."""
    _sweep(105, "few-bins", math=hip.MATH_BF16X3_ALWAYS)


def test_wide_layers():
    """16-130 input channels: staging in chunks, the position-wise weight gradient, two-pass input gradients."""
    _sweep(106, "wide")


def test_residue_classes_forced():
    """Mellin layers per residue class whatever their size."""
    _sweep(107, "any", variant="classes")


def test_half_precision_against_the_checker_on_the_same_half_operands():
    _sweep(108, "any", dtype=np.float16)


def test_accumulate_into_h():
    """Section 1 of the C ABI (h += ...) on one to four bins, transposed layouts drawn at random:
    every word without a tap keeps what the caller put there, bit for bit."""
    rng = np.random.default_rng(109)
    kinds = {"mcorrlcorr": (0, 2), "mconvlconv": (1, 3), "lcorrlcorr": (2, 2), "lconvlconv": (3, 3)}
    done = 0
    t0 = time.time()
    while done < COUNT and time.time() - t0 < SECONDS:
        op = sorted(kinds)[int(rng.integers(4))]
        c_out = int(rng.choice([1, 5, 33, 64])); c_in = int(rng.choice([1, 3, 17, 40])); n = int(rng.integers(1, 4))
        nf = (int(rng.integers(1, 6)), int(rng.integers(1, 5)))
        ng = (int(rng.integers(1, 40)), int(rng.integers(1, 5)))
        nh = (int(rng.integers(1, 50)), int(rng.integers(1, 7)))
        s = tuple(int(v) for v in rng.integers(1, 3, 2)); d = tuple(int(v) for v in rng.integers(1, 3, 2))
        p = tuple(int(v) for v in rng.integers(0, 3, 2)); u = tuple(int(v) for v in rng.integers(1, 3, 2))
        tf, tg, th = (bool(v) for v in rng.integers(0, 2, 3))
        w = rng.standard_normal(c_out * c_in * nf[0] * nf[1]).astype(np.float32)
        x = rng.standard_normal(n * c_in * ng[0] * ng[1]).astype(np.float32)
        h0 = rng.standard_normal(n * c_out * nh[0] * nh[1]).astype(np.float32)
        exp = h0.astype(np.float64)
        oracle.kernel2d(kinds[op], w.astype(np.float64), x.astype(np.float64), exp, c_out, c_in, n, nf, ng, nh,
                        s, d, p, u, tf, tg, th)
        h = to_gpu(h0)
        hip.accumulate(op, to_gpu(w), to_gpu(x), h, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        got = to_np(h)
        layer = (op, c_out, c_in, n, nf, ng, nh, s, d, p, u, tf, tg, th)
        err = np.abs(got.astype(np.float64) - exp)
        assert np.all(err <= 1e-5 * np.abs(exp) + 1e-5 * (c_in * nf[0] * nf[1]) ** 0.5), (done, layer, float(err.max()))
        untouched = exp == h0.astype(np.float64)
        assert np.array_equal(got[untouched], h0[untouched]), (done, layer, "a word without a tap was written")
        done += 1
    print("accumulate: %d calls in %.1f s" % (done, time.time() - t0))
    assert done >= MIN_COUNT


def test_lds_gather_kernels_forced():
    """The vector-ALU gather kernels wherever they apply (few input channels, unit y stride and dilation)."""
    v = _sweep(110, "few-channels", variant="lds-gather")
    assert v.get("lds-gather", 0) >= 20, v


def test_narrow_forward_kernel_forced():
    """The few-channel linear forward kernel on layers of its class however small (the automatic
    choice takes it from 1024 tiles on): partial tiles, partial channel blocks, 1-16 input channels."""
    v = _sweep(111, "narrow-class", math=hip.MATH_BF16X3_ALWAYS, variant="narrow")
    assert v.get("mfma-narrow", 0) >= 40, v


def test_narrow_forward_kernel_relu_and_no_bias():
    """The few-channel linear forward kernel with the fused ReLU and without a bias: bit-identical
    to relu(.) of its own plain result, and to the plain result with a zero bias."""
    rng = np.random.default_rng(112)
    hip.set_math(hip.MATH_BF16X3_ALWAYS)
    hip.set_variant("narrow")
    try:
        for n, c_in, c_out, nf, ng, s, d in ((2, 3, 64, (8, 4), (70, 41), (1, 1), (1, 1)),
                                             (3, 5, 33, (3, 2), (24, 13), (2, 1), (3, 1)),
                                             (1, 8, 70, (2, 4), (14, 12), (1, 1), (2, 1))):
            x = to_gpu(rng.standard_normal((n, c_in) + ng).astype(np.float32))
            w = to_gpu((rng.standard_normal((c_out, c_in) + nf) * 0.2).astype(np.float32))
            b = to_gpu(rng.standard_normal(c_out).astype(np.float32))
            nh = ((ng[0] - d[0] * (nf[0] - 1) - 1) // s[0] + 1, ng[1] - nf[1] + 1)
            dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, (0, 0), (1, 1))
            nan = float("nan")
            plain = torch.full((n, c_out) + nh, nan, device="cuda")
            act = torch.full_like(plain, nan)
            hip.corr2d_forward(hip.AX_LCORR, x, w, b, plain, dims)
            assert hip.last_variant() == "mfma-narrow"
            hip.corr2d_forward(hip.AX_LCORR, x, w, b, act, dims, activation=hip.ACT_RELU)
            assert hip.last_variant() == "mfma-narrow"
            assert torch.equal(act, torch.relu(plain))
            nobias = torch.full_like(plain, nan)
            zero = torch.full_like(plain, nan)
            hip.corr2d_forward(hip.AX_LCORR, x, w, None, nobias, dims)
            hip.corr2d_forward(hip.AX_LCORR, x, w, torch.zeros_like(b), zero, dims)
            assert torch.equal(nobias, zero) and not torch.isnan(nobias).any()
    finally:
        hip.set_variant(None)
        hip.set_math(hip.MATH_BF16X3)
