"""The library's calls can be recorded into a HIP graph (they allocate nothing, never
synchronise, and clear no memory with memset nodes): every replay must reproduce the
eager results bit for bit, with eager work and synchronisations between the replays."""
import pytest
import torch

import _mellin_hip as hip

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", [hip.AX_MCORR, hip.AX_LCORR], ids=["mellin", "linear"])
def test_forward_and_both_gradients_replay_identically(kind):
    torch.manual_seed(1)
    n, c_in, c_out, nf, ng = 4, 3, 64, (8, 4), (128, 41)
    nhx = 16 if kind == hip.AX_MCORR else 121
    nh = (nhx, 38)
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, (1, 1), (1, 1), (0, 0), (1, 1))
    x = torch.randn(n, c_in, *ng, device="cuda")
    w = torch.randn(c_out, c_in, *nf, device="cuda") * 0.1
    b = torch.randn(c_out, device="cuda")
    go = torch.randn(n, c_out, *nh, device="cuda")
    out, gi, gw = torch.empty_like(go), torch.empty_like(x), torch.empty_like(w)
    ws_i = torch.empty(max(hip.lib.mellin_corr2d_backward_input_workspace(kind, 4, *dims), 256),
                       dtype=torch.uint8, device="cuda")
    ws_w = torch.empty(max(hip.lib.mellin_corr2d_backward_weight_workspace(kind, 4, *dims), 256),
                       dtype=torch.uint8, device="cuda")

    def step():
        hip.corr2d_forward(kind, x, w, b, out, dims)
        hip.corr2d_backward_input(kind, w, go, gi, dims, workspace=ws_i, workspace_bytes=ws_i.numel())
        hip.corr2d_backward_weight(kind, x, go, gw, dims, workspace=ws_w, workspace_bytes=ws_w.numel())

    for _ in range(2):
        step()                                            # also grants the kernels their LDS sizes
    torch.cuda.synchronize()
    ref = [t.clone() for t in (out, gi, gw)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for t in (out, gi, gw):
            t.fill_(float("nan"))
        ws_i.fill_(255)
        ws_w.fill_(255)
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip((out, gi, gw), ref):
            assert torch.equal(got, exp), "replay %d differs" % rep
        x2 = torch.randn_like(x)                          # unrelated eager work between replays
        hip.corr2d_forward(kind, x2, w, b, torch.empty_like(out), dims)
        torch.cuda.synchronize()
