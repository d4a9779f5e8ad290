"""Half precision and autocast (the reference's Autocast registration,
ext/torch.cpp:405-447, and its tests, tests/test_mconv.py:814-891).

Through the C ABI: half operands, exact products, fp32 accumulation, one rounding of the
result -- on the f16 matrix cores straight from the half tensors where the tiled kernel
applies ("mfma-f16"), else through fp32 copies of the operands and the fp32 kernels.  The
expected values are the float64 checker on the SAME half-rounded operands, so the only
error left is the final rounding to half (relative 2^-11) plus the fp32 accumulation
(rtol 1e-5, atol 1e-5 * sqrt(fan_in)): asserted as rtol 1e-3, atol 1e-3 * sqrt(fan_in) * 1e-2
-- ten times tighter than the 1e-2 the reference's own autocast tests allow.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
import mconv
from _gpu import to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu

CASES = [
    # kind, n, c_in, c_out, nf, ng, s, d, p, u, r
    ("mcorr", 3, 4, 10, (5, 3), (40, 17), (1, 1), (2, 1), (1, 1), (1, 1), (0, 0)),
    ("lcorr", 2, 3, 64, (8, 4), (60, 41), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),     # fused input gradient underneath
    ("mcorr", 2, 3, 64, (8, 4), (96, 41), (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)),     # tap products underneath
    ("lcorr", 2, 40, 70, (3, 3), (30, 20), (2, 1), (1, 2), (1, 1), (1, 1), (1, 0)),    # many channels
    ("mcorr", 4, 6, 9, (6, 1), (50, 1), (1, 1), (1, 1), (2, 0), (2, 1), (0, 0)),       # 1-D
    ("lcorr", 1, 5, 200, (2, 3), (23, 19), (1, 2), (2, 1), (1, 2), (1, 1), (0, 1)),    # four channel blocks side by side in the weight gradient
    ("mcorr", 3, 2, 100, (3, 2), (31, 3), (2, 1), (1, 1), (1, 0), (1, 1), (3, 0)),     # two; rows of two outputs, twelve columns
]


def _close(got, exp, fan_in, what):
    got = to_np(got.float()).astype(np.float64)
    tol = 1e-3 * np.abs(exp) + 1e-5 * np.sqrt(fan_in)
    bad = np.abs(got - exp) > tol
    assert not bad.any(), "%s: %d of %d off, worst %g" % (what, bad.sum(), bad.size, np.abs(got - exp).max())


@pytest.fixture(params=["auto", "widen"])
def half_path(request):
    """the kernels that read half tensors themselves where they apply, and the copies to fp32 everywhere"""
    hip.set_variant(request.param)
    yield request.param
    hip.set_variant(None)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_half_passes_match_checker_on_the_same_operands(case, half_path):
    kind, n, c_in, c_out, nf, ng, s, d, p, u, r = case
    kind_x = hip.AX_MCORR if kind == "mcorr" else hip.AX_LCORR
    fwd = oracle.mcorrlcorr if kind == "mcorr" else oracle.lcorrlcorr
    bwd = oracle.mcorrlcorr_backward if kind == "mcorr" else oracle.lcorrlcorr_backward
    rng = np.random.default_rng(800 + CASES.index(case))
    x = rng.standard_normal((n, c_in) + ng).astype(np.float16)
    w = (rng.standard_normal((c_out, c_in) + nf) / np.sqrt(c_in * nf[0] * nf[1])).astype(np.float16)
    b = rng.standard_normal(c_out).astype(np.float16)
    x64, w64, b64 = x.astype(np.float64), w.astype(np.float64), b.astype(np.float64)
    exp = fwd(x64, w64, b64, s, d, p, u, r)
    nh = exp.shape[2:]
    assert min(nh) > 0
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
    xg, wg, bg = to_gpu(x), to_gpu(w), to_gpu(b)
    out = torch.full((n, c_out) + nh, float("nan"), dtype=torch.float16, device="cuda")
    hip.corr2d_forward(kind_x, xg, wg, bg, out, dims)
    assert (hip.last_variant() == "mfma-f16") == (half_path == "auto")
    assert (hip.last_math() == hip.MATH_F16) == (half_path == "auto")
    _close(out, exp, c_in * nf[0] * nf[1], "forward %s" % (case,))
    go = rng.standard_normal(exp.shape).astype(np.float16)
    egi, egw, _ = bwd(x64, w64, go.astype(np.float64), s, d, p, u)
    gi = torch.full_like(xg, float("nan"))
    hip.corr2d_backward_input(kind_x, wg, to_gpu(go), gi, dims)
    if half_path == "auto" and CASES.index(case) in (1, 2, 3):
        # the three forms that read half tensors: one kernel (at most three input channels, linear x
        # axis), two passes (few input channels otherwise), the tiled kernel (many)
        assert hip.last_variant() == {1: "mfma-f16-fused", 2: "mfma-f16+fold", 3: "mfma-f16"}[CASES.index(case)]
    _close(gi, egi, c_out * nf[0] * nf[1], "grad_input %s" % (case,))
    gw = torch.full_like(wg, float("nan"))
    hip.corr2d_backward_weight(kind_x, xg, to_gpu(go), gw, dims)
    assert (hip.last_variant() == "mfma-f16") == (half_path == "auto")
    _close(gw, egw, n * nh[0] * nh[1], "grad_weight %s" % (case,))


def test_random_layers_agree_between_the_two_half_paths():
    """Random layers (Mellin and linear, 1-D and 2-D, strides, dilations, paddings, extra
    output rows, one to 260 channels): what the kernels that read half tensors give must be
    what the fp32 kernels give on fp32 copies, up to the rounding of the result to half and
    fp32 summation order."""
    rng = np.random.default_rng(2024)
    seen = {}
    done = 0
    while done < 160:
        mell = bool(rng.integers(2))
        kind_x = hip.AX_MCORR if mell else hip.AX_LCORR
        n = int(rng.integers(1, 6))
        c_in = int(rng.choice([1, 3, 8, 16, 20, 33, 64, 130, 260]))
        c_out = int(rng.choice([3, 16, 33, 64, 70, 130, 260]))
        nf = [(8, 4), (4, 4), (2, 4), (4, 2), (3, 8), (1, 8), (8, 1), (5, 5), (3, 3), (1, 1), (3, 1)][int(rng.integers(11))]
        ng = (int(rng.integers(nf[0], 60)), int(rng.choice([3, 5, 8, 9, 13, 16, 20, 33, 41, 64, 130])))
        if rng.integers(6) == 0:
            nf, ng = (nf[0], 1), (int(rng.integers(nf[0], 300)), 1)
        if ng[1] < nf[1]:
            continue
        s = (int(rng.integers(1, 3)), int(rng.integers(1, 3)) if ng[1] > 1 else 1)
        d = (int(rng.integers(1, 3)), int(rng.integers(1, 3)) if ng[1] > 1 else 1)
        p = (int(rng.integers(0, 4)), int(rng.integers(0, 3)) if ng[1] > 1 else 0)
        r = (int(rng.choice([0, 0, 3, 10])), int(rng.choice([0, 0, 1])) if ng[1] > 1 else 0)
        size_x = mconv.mcorr_valid_size if mell else mconv.lcorr_valid_size
        nh = (size_x(nf[0], ng[0], s[0], d[0], p[0], 1) + r[0],
              mconv.lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], 1) + r[1])
        if min(nh) <= 0 or n * c_out * nh[0] * nh[1] * c_in * nf[0] * nf[1] > 1e9:
            continue
        dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))
        x = to_gpu(rng.standard_normal((n, c_in) + ng).astype(np.float16))
        w = to_gpu((rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float16))
        b = to_gpu(rng.standard_normal(c_out).astype(np.float16))
        go = to_gpu((0.1 * rng.standard_normal((n, c_out) + nh)).astype(np.float16))
        got = {}
        for variant in ("widen", "auto"):
            hip.set_variant(variant)
            try:
                out = torch.full((n, c_out) + nh, float("nan"), dtype=torch.float16, device="cuda")
                gi, gw = torch.full_like(x, float("nan")), torch.full_like(w, float("nan"))
                names = []
                hip.corr2d_forward(kind_x, x, w, b, out, dims)
                names.append(hip.last_variant())
                hip.corr2d_backward_input(kind_x, w, go, gi, dims)
                names.append(hip.last_variant())
                hip.corr2d_backward_weight(kind_x, x, go, gw, dims)
                names.append(hip.last_variant())
                got[variant] = (out.float(), gi.float(), gw.float())
            finally:
                hip.set_variant(None)
            if variant == "auto":
                for pass_, name in zip(("forward", "input", "weight"), names):
                    seen[(pass_, name)] = seen.get((pass_, name), 0) + 1
        fans = (c_in * nf[0] * nf[1], c_out * nf[0] * nf[1], n * nh[0] * nh[1])
        for i, what in enumerate(("out", "grad_input", "grad_weight")):
            ref, res = got["widen"][i], got["auto"][i]
            tol = 2.0 ** -10 * ref.abs() + 2e-5 * fans[i] ** 0.5 * (0.1 if i else 1.0) + 1e-7
            assert bool(((ref - res).abs() <= tol).all()), (what, mell, n, c_in, c_out, nf, ng, s, d, p, r)
        done += 1
    # the sample exercised every kernel that reads half tensors
    assert seen.get(("forward", "mfma-f16"), 0) > 100 and seen.get(("weight", "mfma-f16"), 0) > 100
    assert seen.get(("input", "mfma-f16"), 0) > 30 and seen.get(("input", "mfma-f16+fold"), 0) + seen.get(("input", "mfma-f16-filter-rows+fold"), 0) > 10, seen
    assert seen.get(("input", "mfma-f16-fused"), 0) > 3, seen


def test_workspace_is_required_and_sized():
    dims = hip._dims(2, 3, 8, (4, 2), (20, 9), (4, 8), (1, 1), (1, 1), (0, 0), (1, 1))
    x = torch.randn(2, 3, 20, 9, device="cuda").half()
    w = torch.randn(8, 3, 4, 2, device="cuda").half()
    out = torch.empty(2, 8, 4, 8, device="cuda", dtype=torch.float16)
    # the kernel that reads half tensors needs nothing for a filter this small
    assert hip.lib.mellin_corr2d_forward_f16_workspace(hip.AX_MCORR, *dims) == 0
    hip.set_variant("widen")
    try:
        _workspace_checks(dims, x, w, out)
    finally:
        hip.set_variant(None)


def _workspace_checks(dims, x, w, out):
    need = hip.lib.mellin_corr2d_forward_f16_workspace(hip.AX_MCORR, *dims)
    assert need >= 4 * (x.numel() + w.numel() + out.numel())
    small = torch.empty(need - 1, dtype=torch.uint8, device="cuda")
    rc = hip.lib.mellin_corr2d_forward_f16(hip.AX_MCORR, x.data_ptr(), w.data_ptr(), None, *dims, out.data_ptr(),
                                           small.data_ptr(), need - 1, None)
    assert rc == 3 and "workspace" in hip.last_error()
    with pytest.raises(RuntimeError, match="share one dtype"):
        hip.corr2d_forward(hip.AX_MCORR, x, w.float(), None, out, dims)


# ---- autocast: the reference's tests (tests/test_mconv.py:814-891), reduced in size ----
def test_autocast_mcorrlcorr_func():
    n, c_in, c_out, t_in, f_in, t_k, f_k = 16, 16, 64, 64, 32, 8, 4
    input = torch.rand(n, c_in, t_in, f_in, device="cuda", dtype=torch.half).float()
    weight = torch.rand(c_out, c_in, t_k, f_k, dtype=torch.half, device="cuda").float()
    bias = torch.rand(c_out, device="cuda", dtype=torch.half).float()
    out_a = mconv.mcorrlcorr(input, weight, bias).half()
    with torch.autocast("cuda"):
        out_b = mconv.mcorrlcorr(input, weight, bias)
    assert out_b.dtype == torch.half
    assert torch.allclose(out_a, out_b, rtol=1e-2, atol=1e-2)
    # here the two differ by the output rounding alone
    assert torch.allclose(out_a.float(), out_b.float(), rtol=2e-3, atol=1e-3)


def test_autocast_mcorr1d_func():
    n, c_in, c_out, t_in, t_k = 32, 16, 64, 128, 16
    input = torch.rand(n, c_in, t_in, device="cuda", dtype=torch.half).float()
    weight = torch.rand(c_out, c_in, t_k, dtype=torch.half, device="cuda").float()
    bias = torch.rand(c_out, device="cuda", dtype=torch.half).float()
    out_a = mconv.mcorr1d(input, weight, bias).half()
    with torch.autocast("cuda"):
        out_b = mconv.mcorr1d(input, weight, bias)
    assert out_b.dtype == torch.half
    assert torch.allclose(out_a, out_b, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("two_d", [False, True], ids=["mcorr1d", "mcorrlcorr"])
def test_autocast_layer_trains_with_a_grad_scaler(two_d):
    torch.manual_seed(3)
    if two_d:
        layer = mconv.MCorrLCorr(16, 8, (4, 2)).cuda()
        input = torch.randn(32, 16, 16, 8, device="cuda")
    else:
        layer = mconv.MCorr1d(16, 8, 8).cuda()
        input = torch.randn(32, 16, 16, device="cuda")
    before = [p_.detach().clone() for p_ in layer.parameters()]
    optimizer = torch.optim.Adam(layer.parameters())
    scaler = torch.amp.GradScaler("cuda", init_scale=128.0)     # 65536, the default, overflows half at once
    optimizer.zero_grad()
    with torch.autocast("cuda"):
        output = layer(input)
        assert output.dtype == torch.half
        loss = output.float().mean()                    # (a plain sum overflows half in the bias gradient)
    scaler.scale(loss).backward()
    for p_ in layer.parameters():
        assert p_.grad is not None and p_.grad.dtype == torch.float32 and torch.isfinite(p_.grad).all()
    # the same gradients, unscaled, as the fp32 layer gives (to half accuracy)
    ref = [torch.autograd.grad(layer(input).mean(), p_)[0] for p_ in layer.parameters()]
    scale = scaler.get_scale()
    for p_, g_ in zip(layer.parameters(), ref):
        assert torch.allclose(p_.grad / scale, g_, rtol=2e-2, atol=2e-2 * float(g_.abs().max()))
    scaler.step(optimizer)
    scaler.update()
    assert any(not torch.equal(a, b_) for a, b_ in zip(before, layer.parameters()))


def test_autocast_column_ops():
    x = torch.randn(3, 2, 30, 11, device="cuda")
    full = mconv.spec2col(x.half().float(), (4, 3))
    with torch.autocast("cuda"):
        cols = mconv.spec2col(x, (4, 3))
    assert cols.dtype == torch.half
    assert torch.equal(cols.float(), full)               # a gather moves values unchanged


@pytest.mark.parametrize("shape", [
    # (kind, n, c_in, c_out, nf, ng): few channels (forward stores half itself), many (so does the input gradient)
    ("lcorr", 3, 3, 40, (8, 4), (70, 41)), ("mcorr", 2, 3, 64, (8, 4), (64, 41)),
    ("lcorr", 2, 48, 70, (3, 3), (30, 21)), ("mcorr", 2, 40, 33, (4, 4), (40, 5)),
], ids=["lcorr-few", "mcorr-few", "lcorr-many", "mcorr-many"])
def test_half_results_are_the_fp32_results_rounded_once(shape, half_path):
    """Through the fp32 copies the half entry points compute as the fp32 ones do on the
    widened operands: whichever kernel stores the result, it must equal the fp32 result
    rounded to nearest even, bit for bit.  The f16 matrix instructions sum the same exact
    products in another order: their fp32 sums differ from the fp32 kernels' in the last
    bits, which moves a result to the neighbouring half value only where the sum lies
    that close to a rounding boundary -- in under 1 % of the results."""
    kind, n, c_in, c_out, nf, ng = shape
    kind_x = hip.AX_MCORR if kind == "mcorr" else hip.AX_LCORR
    op = mconv.mcorrlcorr if kind == "mcorr" else mconv.lcorrlcorr
    gen = torch.Generator().manual_seed(11)
    x = torch.randn((n, c_in) + ng, generator=gen).half().cuda()
    w = (torch.randn((c_out, c_in) + nf, generator=gen) * (c_in * nf[0] * nf[1]) ** -0.5).half().cuda()
    b = torch.randn(c_out, generator=gen).half().cuda()
    def same(got, ref32, fan_in):
        exp = ref32.half()
        if half_path == "widen":
            return torch.equal(got, exp)
        # half the spacing of half values at the result, plus what fp32 accumulation may differ by
        half_step = exp.float().abs().clamp_min(2.0 ** -14) * 2.0 ** -11
        close = (got.float() - ref32).abs() <= 1.001 * half_step + 1e-5 * fan_in ** 0.5
        return bool(close.all()) and float((got != exp).float().mean()) < 0.01

    ref = op(x.float(), w.float(), b.float())
    out = op(x, w, b)
    assert out.dtype == torch.float16 and same(out, ref, c_in * nf[0] * nf[1])
    nh = tuple(ref.shape[2:])
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    go = torch.randn(ref.shape, generator=gen).half().cuda()
    gi32 = torch.empty_like(x, dtype=torch.float32)
    hip.corr2d_backward_input(kind_x, w.float(), go.float(), gi32, dims)
    gi16 = torch.empty_like(x)
    hip.corr2d_backward_input(kind_x, w, go, gi16, dims)
    assert same(gi16, gi32, c_out * nf[0] * nf[1])


def test_half_views_at_odd_offsets():
    """Half tensors that start at any even address (a slice of a flat buffer, a cat gradient):
    the copies between half and fp32 then go element by element instead of 16 bytes at a time.
    All three passes must give bit for bit what the same operands give from aligned storage."""
    kind, n, c_in, c_out, nf, ng, s, d, p, u, r = CASES[1]
    rng = np.random.default_rng(42)
    x = torch.from_numpy(rng.standard_normal((n, c_in) + ng).astype(np.float16))
    w = torch.from_numpy((rng.standard_normal((c_out, c_in) + nf) * 0.1).astype(np.float16))
    b = torch.from_numpy(rng.standard_normal(c_out).astype(np.float16))
    nh = (mconv.lcorr_valid_size(nf[0], ng[0]), mconv.lcorr_valid_size(nf[1], ng[1]))
    go = torch.from_numpy(rng.standard_normal((n, c_out) + nh).astype(np.float16))
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)

    def shifted(t, off):
        """the same values in storage that starts `off` halves past a 256-byte boundary"""
        flat = torch.empty(t.numel() + 8, dtype=torch.float16, device="cuda")
        view = flat[off:off + t.numel()].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == (2 * off) % 16
        return view

    def run(off):
        xg, wg, bg, gog = (shifted(t, off) for t in (x, w, b, go))
        out = shifted(torch.zeros((n, c_out) + nh, dtype=torch.float16), off)
        gi = shifted(torch.zeros_like(x), off)
        gw = shifted(torch.zeros_like(w), off)
        hip.corr2d_forward(hip.AX_LCORR, xg, wg, bg, out, dims)
        hip.corr2d_backward_input(hip.AX_LCORR, wg, gog, gi, dims)
        hip.corr2d_backward_weight(hip.AX_LCORR, xg, gog, gw, dims)
        return out.clone(), gi.clone(), gw.clone()

    for variant in ("auto", "widen"):
        hip.set_variant(variant)
        try:
            aligned = run(0)
            for off in (1, 3):
                for a, c in zip(aligned, run(off)):
                    assert torch.equal(a, c)
        finally:
            hip.set_variant(None)


def test_wide_layers_read_their_filter_from_fragments_in_the_workspace():
    """Layers whose channels are staged in several chunks: the filter's fragments are made once
    per call in the workspace (the only scratch memory the call needs), for the forward pass
    and, with many input channels, for the input gradient, Mellin and linear."""
    for kind_x, op in ((hip.AX_LCORR, mconv.lcorrlcorr), (hip.AX_MCORR, mconv.mcorrlcorr)):
        n, c_in, c_out, nf, ng, s, d, p, u = 3, 150, 130, (3, 3), (40, 23), (1, 1), (2, 1), (2, 1), (1, 1)
        gen = torch.Generator().manual_seed(5)
        x = torch.randn((n, c_in) + ng, generator=gen).half().cuda()
        w = (torch.randn((c_out, c_in) + nf, generator=gen) * (c_in * 9) ** -0.5).half().cuda()
        b = torch.randn(c_out, generator=gen).half().cuda()
        ref = op(x.float(), w.float(), b.float(), s, d, p, u)
        nh = tuple(ref.shape[2:])
        dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
        need = hip.lib.mellin_corr2d_forward_f16_workspace(kind_x, *dims)
        assert 0 < need <= 2 * 2 * w.numel() * 2          # the filter once, padded to 16 taps per chunk and whole tiles
        out = op(x, w, b, s, d, p, u)
        assert hip.last_variant() == "mfma-f16"
        tol = 2.0 ** -10 * ref.abs().clamp_min(2.0 ** -14) + 1e-5 * (c_in * 9) ** 0.5
        assert bool(((out.float() - ref).abs() <= tol).all())
        go = torch.randn(ref.shape, generator=gen).half().cuda()
        gi32 = torch.empty_like(x, dtype=torch.float32)
        hip.corr2d_backward_input(kind_x, w.float(), go.float(), gi32, dims)
        gi = torch.empty_like(x)
        hip.corr2d_backward_input(kind_x, w, go, gi, dims)
        # (this Mellin layer keeps fewer rows than it is given: the two-pass form, as in fp32)
        assert hip.last_variant() in (("mfma-f16",) if kind_x == hip.AX_LCORR else ("mfma-f16+fold", "mfma-f16-filter-rows+fold"))
        if kind_x == hip.AX_LCORR:
            assert 0 < hip.lib.mellin_corr2d_backward_input_f16_workspace(kind_x, *dims) <= 2 * 2 * w.numel() * 2
        tol = 2.0 ** -10 * gi32.abs().clamp_min(2.0 ** -14) + 1e-5 * (c_out * 9) ** 0.5
        assert bool(((gi.float() - gi32).abs() <= tol).all())
        # too little scratch memory is an error, not a slower path
        small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
        rc = hip.lib.mellin_corr2d_forward_f16(kind_x, x.data_ptr(), w.data_ptr(), b.data_ptr(), *dims,
                                               out.data_ptr(), small.data_ptr(), need - 16, None)
        assert rc == 3 and "workspace" in hip.last_error()


def test_subnormal_half_operands_are_not_flushed():
    """Products of subnormal half values with large ones are ordinary numbers; the f16 matrix
    instructions must take such operands as they are."""
    n, c_in, c_out, nf, ng = 1, 2, 32, (2, 2), (9, 40)
    x = torch.full((n, c_in) + ng, 2.0 ** -20, dtype=torch.float16, device="cuda")      # subnormal: below 2^-14
    x[0, 1] = 3 * 2.0 ** -24
    w = torch.full((c_out, c_in) + nf, 1024.0, dtype=torch.float16, device="cuda")
    out = mconv.lcorrlcorr(x, w, None)
    assert hip.last_variant() == "mfma-f16"
    exp = 4 * 1024.0 * (2.0 ** -20 + 3 * 2.0 ** -24)
    assert torch.equal(out, torch.full_like(out, exp))
