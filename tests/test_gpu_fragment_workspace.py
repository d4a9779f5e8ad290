"""Layers staged in chunks multiply on the bf16 matrix cores from the filter cut into bf16
parts.  With scratch memory that copy is made once per call (forward:
mellin_corr2d_forward_ws_f32; input gradient: the workspace it already takes), without it
every workgroup cuts the filter itself.  Both ways build the same fragments and multiply in
the same order: the results must agree bit for bit, and with the float64 checker to
rtol 1e-5 / atol 1e-5 * sqrt(fan_in)."""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu

CASES = [
    # (kind, n, c_in, c_out, nf, ng, s, d, p): each above the size from which layers staged in chunks
    # take the bf16 cores (0.8 GMAC)
    (hip.AX_LCORR, 4, 160, 96, (3, 3), (40, 41), (1, 1), (2, 1), (2, 1)),     # a short last chunk
    (hip.AX_LCORR, 6, 96, 128, (4, 4), (48, 20), (1, 1), (1, 1), (1, 1)),
    (hip.AX_MCORR, 8, 128, 128, (4, 4), (120, 14), (1, 1), (1, 1), (1, 1)),   # wide Mellin: two-pass input gradient
    (hip.AX_MCORR, 6, 96, 128, (3, 4), (200, 24), (2, 1), (1, 1), (1, 2)),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-%dx%d" % ("mellin" if c[0] == hip.AX_MCORR else "linear", c[2], c[3]))
def test_with_and_without_scratch_memory(case):
    import mconv
    kind, n, c_in, c_out, nf, ng, s, d, p = case
    u = (1, 1)
    valid_x = mconv.mcorr_valid_size if kind == hip.AX_MCORR else mconv.lcorr_valid_size
    nh = (valid_x(nf[0], ng[0], s[0], d[0], p[0], 1), mconv.lcorr_valid_size(nf[1], ng[1], s[1], d[1], p[1], 1))
    rng = np.random.default_rng(7)
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = (rng.standard_normal((c_out, c_in) + nf) * (c_in * nf[0] * nf[1]) ** -0.5).astype(np.float32)
    b = rng.standard_normal(c_out).astype(np.float32)
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, u)
    xg, wg, bg, gog = to_gpu(x), to_gpu(w), to_gpu(b), to_gpu(go)
    hip.set_math(hip.MATH_BF16X3)

    need = hip.lib.mellin_corr2d_forward_workspace(kind, 4, *dims)
    assert need > 0, "the case is meant to be staged in chunks"
    out_ws = torch.full(go.shape, float("nan"), device="cuda")
    hip.corr2d_forward(kind, xg, wg, bg, out_ws, dims)             # allocates and passes the scratch memory
    assert hip.last_variant() == "mfma" and hip.last_math() == hip.MATH_BF16X3
    out_plain = torch.full(go.shape, float("nan"), device="cuda")
    rc = hip.lib.mellin_corr2d_forward_act_f32(kind, hip.ACT_NONE, hip._dp(xg), hip._dp(wg), hip._dp(bg), *dims,
                                               hip._dp(out_plain), hip._stream(xg.device))
    assert rc == 0 and hip.last_math() == hip.MATH_BF16X3
    assert torch.equal(out_ws, out_plain)
    op = oracle.mcorrlcorr if kind == hip.AX_MCORR else oracle.lcorrlcorr
    ref = op(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64), s, d, p, u, (0, 0))
    assert_close(out_ws, ref, c_in * nf[0] * nf[1])
    # too little scratch memory is refused, none at all as well
    small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
    rc = hip.lib.mellin_corr2d_forward_ws_f32(kind, hip.ACT_NONE, hip._dp(xg), hip._dp(wg), hip._dp(bg), *dims,
                                              hip._dp(out_plain), hip._dp(small), need - 16, hip._stream(xg.device))
    assert rc != 0 and "workspace" in hip.lib.mellin_last_error().decode()

    # input gradient: with the workspace the query asks for, and (gather form only) without
    need_in = hip.lib.mellin_corr2d_backward_input_workspace(kind, 4, *dims)
    assert need_in > 0
    gi_ws = torch.full(x.shape, float("nan"), device="cuda")
    hip.corr2d_backward_input(kind, wg, gog, gi_ws, dims)
    variant = hip.last_variant()
    assert variant in ("mfma", "mfma+fold", "mfma-filter-rows+fold") and hip.last_math() == hip.MATH_BF16X3
    if variant == "mfma":
        gi_plain = torch.full(x.shape, float("nan"), device="cuda")
        rc = hip.lib.mellin_corr2d_backward_input_f32(kind, hip._dp(wg), hip._dp(gog), *dims, hip._dp(gi_plain),
                                                      None, 0, hip._stream(xg.device))
        assert rc == 0
        assert torch.equal(gi_ws, gi_plain)
    bwd = oracle.mcorrlcorr_backward if kind == hip.AX_MCORR else oracle.lcorrlcorr_backward
    gi_ref = bwd(x.astype(np.float64), w.astype(np.float64), go.astype(np.float64), s, d, p, u)[0]
    assert_close(gi_ws, gi_ref, c_out * nf[0] * nf[1])
