"""The allocation-free weight gradient (mellin_corr2d_backward_weight_static_f32): same
result, bit for bit, as mellin_corr2d_backward_weight_f32 with a caller's workspace, on
two calls in a row that share the library's static scratch array, the second on a smaller
layer; no device memory is allocated on the way; layers past the array's size are refused.
Both sides go through the C ABI.
"""
import numpy as np
import pytest
import torch

import _mellin_hip as hip
from _gpu import assert_close, to_gpu
from oracle import oracle

pytestmark = pytest.mark.gpu


def _layer(seed, n, c_in, c_out, nf, ng, kind_x):
    rng = np.random.default_rng(seed)
    fwd = oracle.mcorrlcorr if kind_x == hip.AX_MCORR else oracle.lcorrlcorr
    x = rng.standard_normal((n, c_in) + ng).astype(np.float32)
    w = rng.standard_normal((c_out, c_in) + nf).astype(np.float32)
    nh = fwd(x, w, None, (1, 1), (1, 1), (0, 0), (1, 1), (0, 0)).shape[2:]
    go = rng.standard_normal((n, c_out) + nh).astype(np.float32)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    return x, go, w.shape, dims, nh


def test_static_scratch_matches_workspace_entry_point_twice():
    assert hip.lib.mellin_static_scratch_bytes() == 16 << 20
    # the benchmark's layer on 8 utterances, then a smaller layer of the other kind: the second
    # call finds the first one's partial sums in the array
    cases = [(1, 8, 3, 64, (8, 4), (512, 41), hip.AX_LCORR), (2, 3, 5, 20, (3, 3), (60, 23), hip.AX_MCORR)]
    for seed, n, c_in, c_out, nf, ng, kind_x in cases:
        x, go, w_shape, dims, nh = _layer(seed, n, c_in, c_out, nf, ng, kind_x)
        need = hip.lib.mellin_corr2d_backward_weight_workspace(kind_x, 4, *dims)
        assert 0 < need <= hip.lib.mellin_static_scratch_bytes(), need
        xg, gog = to_gpu(x), to_gpu(go)
        ref = torch.full(w_shape, float("nan"), dtype=torch.float32, device="cuda")
        hip.corr2d_backward_weight(kind_x, xg, gog, ref, dims)
        got = torch.full(w_shape, float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        hip.corr2d_backward_weight_static(kind_x, xg, gog, got, dims)
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
        assert torch.equal(got, ref), (seed, (got - ref).abs().max().item())
        # and both are the checker's weight gradient
        bwd = oracle.mcorrlcorr_backward if kind_x == hip.AX_MCORR else oracle.lcorrlcorr_backward
        w0 = np.zeros(w_shape)
        _, exp, _ = bwd(x.astype(np.float64), w0, go.astype(np.float64), (1, 1), (1, 1), (0, 0), (1, 1))
        assert_close(got, exp, n * nh[0] * nh[1], "static weight gradient, case %d" % seed)


def test_prepare_does_the_lookup_alone():
    """mellin_static_scratch_prepare(): the address lookup without a layer (what a caller runs
    before capturing a graph); it may be called any number of times."""
    assert hip.lib.mellin_static_scratch_prepare() == 0
    assert hip.lib.mellin_static_scratch_prepare() == 0


def test_layer_beyond_the_static_array_is_refused():
    # 1024 x 272 channels of 4 x 4 taps: the partial sums of one split alone pass 16 MiB
    n, c_in, c_out, nf, ng = 1, 272, 1024, (4, 4), (8, 8)
    nh = (5, 5)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    need = hip.lib.mellin_corr2d_backward_weight_workspace(hip.AX_LCORR, 4, *dims)
    assert need > hip.lib.mellin_static_scratch_bytes(), need
    x = torch.zeros((n, c_in) + ng, device="cuda")
    go = torch.zeros((n, c_out) + nh, device="cuda")
    gw = torch.zeros((c_out, c_in) + nf, device="cuda")
    with pytest.raises(RuntimeError, match="static array holds"):
        hip.corr2d_backward_weight_static(hip.AX_LCORR, x, go, gw, dims)
