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


def test_pointwise_layers_are_capturable():
    """log compression + dilation lift with eps = exp(log_eps), tau = exp(log_tau) computed on the
    device: the values reach the kernels through device memory, so neither the forward nor the
    backward pass waits for the device, and both can be recorded and replayed."""
    import layers
    torch.manual_seed(3)
    x = torch.randn(6, 3, 50, 17, device="cuda")
    gy = torch.randn_like(x)
    log_eps = torch.tensor(-1.0, device="cuda", requires_grad=True)
    log_tau = torch.tensor(0.3, device="cuda", requires_grad=True)
    y, gx = torch.empty_like(x), torch.empty_like(x)
    g_eps, g_tau = torch.empty((), device="cuda"), torch.empty((), device="cuda")

    def step():
        xi = x.detach().requires_grad_(True)
        out = layers.log_compression_lift(xi, log_eps.exp(), log_tau.exp(), 2)
        a, b, c = torch.autograd.grad(out, (xi, log_eps, log_tau), gy)
        y.copy_(out.detach()); gx.copy_(a); g_eps.copy_(b); g_tau.copy_(c)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                        # warm-up off the default stream, as capture requires
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ref = [t.clone() for t in (y, gx, g_eps, g_tau)]
    eps, tau = float(log_eps.detach().exp()), float(log_tau.detach().exp())
    t = torch.arange(1, 51, device="cuda", dtype=torch.float32).view(1, 1, 50, 1)
    torch.testing.assert_close(ref[0], t ** tau * torch.log(eps + x.abs()), rtol=1e-5, atol=1e-5)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        for buf in (y, gx, g_eps, g_tau):
            buf.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip((y, gx, g_eps, g_tau), ref):
            assert torch.equal(got, exp), "replay %d differs" % rep
        layers.log_compression(torch.randn_like(x), torch.tensor(0.5, device="cuda"))   # eager work in between
        torch.cuda.synchronize()
