"""The model-style convolution stack (conv_stack.ConvStack) end to end on the GPU.

* geometry: layer output sizes follow the reference's rule (models.py:292-327:
  every layer's output is input // factor, whatever the kernel);
* parity: forward output and every gradient of a reduced stack against the same
  stack evaluated with the CPU checker in float64 (checker ops wrapped in
  torch.autograd.Function, ReLU / max-pool by torch on the CPU);
* the full-size 10-layer stacks of BASELINE config 5 (3 -> 256 channels, 4x4
  kernels, ReLU, frequency pools, batch 32, 780 x 41, Linear -> 62
  log-probabilities), Mellin and linear: one forward + backward of the whole
  model, then EVERY layer's forward output, input gradient and weight gradient
  of that run against the CPU checker on the layer's own captured input and
  upstream gradient (utterance and channel slices), at the operator tolerance
  rtol 1e-5 / atol 1e-5 * sqrt(fan_in);
* the full-size Mellin stack is finite and run-to-run identical.

Tolerance of the end-to-end comparison of the reduced stack: it compounds five
layers, so outputs and gradients are held to 1e-4 of the largest magnitude of
the tensor compared; per-layer comparisons use the operator tolerance.
"""
import numpy as np
import pytest
import torch

import mconv
from conv_stack import ConvStack, ConvStackParams, FrameClassifier, layer_plan
from _gpu import assert_close, f64, to_gpu, to_np
from oracle import oracle

pytestmark = pytest.mark.gpu


class _CheckerCorr(torch.autograd.Function):
    """A correlation layer evaluated by the CPU checker (float64 numpy)."""

    @staticmethod
    def forward(ctx, x, w, b, kind, s, d, p, r):
        fwd = oracle.mcorrlcorr if kind == "mcorrlcorr" else oracle.lcorrlcorr
        ctx.save_for_backward(x, w)
        ctx.args = (kind, s, d, p)
        return torch.from_numpy(fwd(x.numpy(), w.numpy(), b.numpy(), s, d, p, 1, r))

    @staticmethod
    def backward(ctx, go):
        x, w = ctx.saved_tensors
        kind, s, d, p = ctx.args
        bwd = oracle.mcorrlcorr_backward if kind == "mcorrlcorr" else oracle.lcorrlcorr_backward
        gi, gw, gb = bwd(x.numpy(), w.numpy(), np.ascontiguousarray(go.numpy()), s, d, p, 1)
        return (torch.from_numpy(np.ascontiguousarray(gi)), torch.from_numpy(np.ascontiguousarray(gw)),
                torch.from_numpy(np.ascontiguousarray(gb)), None, None, None, None, None)


def _checker_stack(stack, x64, params64):
    h = x64
    for lay, (w, b) in zip(stack.plan, params64):
        h = torch.relu(_CheckerCorr.apply(h, w, b, lay["kind"], lay["s"], lay["d"], lay["p"], lay["r"]))
        if lay["pool"]:
            h = torch.nn.functional.max_pool2d(h, (1, 2))
    return h


def _close(got, exp, what):
    exp = exp.numpy() if isinstance(exp, torch.Tensor) else exp
    got = to_np(got).astype(np.float64)
    scale = max(float(np.abs(exp).max()), 1e-30)
    np.testing.assert_allclose(got, exp, rtol=0, atol=1e-4 * scale, err_msg=what)


@pytest.mark.parametrize("mellin", [True, False], ids=["mellin", "linear"])
def test_layer_sizes_follow_the_reference_rule(mellin):
    p = ConvStackParams(layers=6, mellin=mellin, kernel_time=5, kernel_freq=3, initial_channels=4,
                        factor_schedule=2, channel_factor=2, time_factor=2, freq_factor=2, in_channels=1)
    x, y = 96, 41
    plan = layer_plan(p, x, y)
    for no, lay in enumerate(plan, 1):
        on = no % 2 == 0
        if mellin:
            x, y = (max(x // 2, 1), max(y // 2, 1)) if on else (x, y)
        else:
            px, py = lay["p"]
            x = (x + 2 * px - 5) // lay["s"][0] + 1
            y = (y + 2 * py - 3) // lay["s"][1] + 1
        assert lay["out_size"] == (x, y), (no, lay)
        assert lay["out_channels"] == 4 * 2 ** (no // 2)
    stack = ConvStack(96, 41, p).cuda()
    out = stack(torch.randn(2, 1, 96, 41, device="cuda"))
    assert tuple(out.shape) == (2, stack.out_channels) + stack.out_size


@pytest.mark.parametrize("mellin", [True, False], ids=["mellin", "linear"])
def test_reduced_stack_matches_checker(mellin):
    p = ConvStackParams(layers=5, mellin=mellin, kernel_time=4, kernel_freq=4, initial_channels=6,
                        factor_schedule=3, channel_factor=2, time_factor=2 if not mellin else 1,
                        freq_factor=1, in_channels=3, freq_pool_after=(3,), seed=4)
    stack = ConvStack(40, 21, p).cuda()
    gen = torch.Generator().manual_seed(4)
    x = torch.randn(2, 3, 40, 21, generator=gen)
    xg = x.cuda().requires_grad_(True)
    out = stack(xg)
    go = torch.randn(out.shape, generator=gen)
    out.backward(go.cuda())

    x64 = x.double().requires_grad_(True)
    params64 = [(c.weight.detach().cpu().double().requires_grad_(True),
                 c.bias.detach().cpu().double().requires_grad_(True)) for c in stack.convs]
    exp = _checker_stack(stack, x64, params64)
    assert tuple(out.shape) == tuple(exp.shape)
    exp.backward(go.double())
    _close(out, exp.detach(), "stack output")
    _close(xg.grad, x64.grad, "grad_input")
    for no, (conv, (w, b)) in enumerate(zip(stack.convs, params64), 1):
        _close(conv.weight.grad, w.grad, "grad_weight layer %d" % no)
        _close(conv.bias.grad, b.grad, "grad_bias layer %d" % no)


def _cfg5_params(mellin):
    return ConvStackParams(layers=10, mellin=mellin, kernel_time=4, kernel_freq=4, initial_channels=32,
                           factor_schedule=3, channel_factor=2, time_factor=1, freq_factor=1, in_channels=3,
                           freq_pool_after=(3, 6, 9), seed=4)


def _unit(a, b):
    """1 / (rms(a) * rms(b)): the scale at which sums of products of a and b meet the
    tolerance's assumption of unit-scale operands (atol 1e-5 * sqrt(fan_in))."""
    ra = float(np.sqrt(np.mean(np.square(a, dtype=np.float64))))
    rb = float(np.sqrt(np.mean(np.square(b, dtype=np.float64))))
    return 1.0 / max(ra * rb, 1e-30)


def _cfg5_batch():
    gen = torch.Generator().manual_seed(4)
    lens = torch.randint(100, 781, (32,), generator=gen)
    x = torch.randn(32, 3, 780, 41, generator=gen)
    x = x * (torch.arange(780)[None, :] < lens[:, None])[:, None, :, None]     # zero past each length
    targets = torch.randint(0, 62, (32, 780), generator=gen)
    return x, lens, targets


@pytest.mark.parametrize("mellin", [True, False], ids=["mellin", "linear"])
def test_full_size_model_every_layer_matches_checker(mellin):
    """BASELINE config 5 as stated: ten layers 3 -> 256 channels, 4 x 4 kernels, ReLU, frequency
    max-pool 2 after layers 3, 6 and 9, linear projection to 62 log-probabilities, batch 32 of
    up to 780 frames x 41 bins, seed 4.  One forward + backward of the model at full size;
    then each layer of THAT run is checked on its own: its captured input and the captured
    gradient of its output go through the checker, on two utterances (forward: all output
    channels of narrow layers, sixteen spread ones of wide layers; input gradient: all
    channels) and, for the weight gradient, on a spread of channel pairs over all 32
    utterances (float64 checker: the sums run over up to a million terms).  Activations and
    gradients deep in the model are far from unit scale, so every comparison is made after
    scaling by 1 / (rms of the one operand x rms of the other), the scale the tolerance
    rtol 1e-5 / atol 1e-5 * sqrt(fan_in) is stated for."""
    stack = ConvStack(780, 41, _cfg5_params(mellin)).cuda()
    assert [lay["out_channels"] for lay in stack.plan] == [32, 32, 64, 64, 64, 128, 128, 128, 256, 256]
    model = FrameClassifier(stack, 62).cuda()
    x, lens, targets = _cfg5_batch()
    seen = {}

    def keep(no):
        def hook(module, inputs, output):
            seen[no] = dict(x=inputs[0], out=output)
            output.register_hook(lambda g, no=no: seen[no].__setitem__("g_out", g))
            if inputs[0].requires_grad:
                inputs[0].register_hook(lambda g, no=no: seen[no].__setitem__("g_in", g))
        return hook

    for no, conv in enumerate(stack.convs):
        conv.register_forward_hook(keep(no))
    xg = x.cuda().requires_grad_(True)
    logp = model(xg)
    t_out = stack.out_size[0]
    assert tuple(logp.shape) == (32, t_out, 62)
    torch.testing.assert_close(logp.exp().sum(-1), torch.ones(32, t_out, device="cuda"), rtol=1e-4, atol=1e-4)
    frame_ok = (torch.arange(t_out)[None, :] < lens[:, None]).cuda()
    loss = -(logp.gather(2, targets[:, :t_out, None].cuda()).squeeze(2) * frame_ok).sum() / frame_ok.sum()
    loss.backward()
    torch.cuda.synchronize()
    assert bool(torch.isfinite(loss)) and bool(torch.isfinite(xg.grad).all())

    nb = [1, 22]
    for no, (lay, conv) in enumerate(zip(stack.plan, stack.convs)):
        rec = seen[no]
        fwd = oracle.mcorrlcorr if lay["kind"] == "mcorrlcorr" else oracle.lcorrlcorr
        bwd = oracle.mcorrlcorr_backward if lay["kind"] == "mcorrlcorr" else oracle.lcorrlcorr_backward
        s, d, p, r = lay["s"], lay["d"], lay["p"], lay["r"]
        c_in, c_out = lay["in_channels"], lay["out_channels"]
        w, b = to_np(conv.weight), to_np(conv.bias)
        xin = to_np(rec["x"][nb])
        out = rec["out"]                                             # after the fused ReLU
        assert tuple(out.shape[:2]) == (32, c_out) and float((out == 0).float().mean()) > 0.05
        what = "%s layer %d (%d -> %d, %s)" % (lay["kind"], no + 1, c_in, c_out, tuple(out.shape[2:]))
        # forward, ReLU included
        co = list(range(c_out)) if c_out <= 64 else list(range(3, c_out, c_out // 16))
        exp = np.maximum(fwd(xin, w[co], b[co], s, d, p, 1, r), 0)
        k = _unit(xin, w)
        assert_close(out[nb][:, co] * k, exp * k, c_in * 16, what + " forward")
        # the gradient that reaches the correlation: zero where the ReLU clamped
        g_pre = rec["g_out"] * (out > 0)
        # input gradient of the two utterances, every input channel
        if "g_in" in rec or no == 0:
            got = xg.grad if no == 0 else rec["g_in"]
            gn = to_np(g_pre[nb])
            gi, _, _ = bwd(xin, w, gn, s, d, p, 1)
            k = _unit(w, gn)
            assert_close(got[nb] * k, gi * k, c_out * 16, what + " grad_input")
        # weight gradient over the whole batch, a spread of channel pairs
        cos = sorted({0, c_out // 3, c_out - 1})
        cis = sorted({0, c_in // 2, c_in - 1})
        xs = np.ascontiguousarray(to_np(rec["x"][:, cis]))
        gs = np.ascontiguousarray(to_np(g_pre[:, cos]))
        _, gw, gb = bwd(*f64(xs, w[cos][:, cis], gs), s, d, p, 1)
        positions = 32 * out.shape[2] * out.shape[3]
        k = _unit(xs, gs)
        assert_close(conv.weight.grad[cos][:, cis] * k, gw * k, positions, what + " grad_weight")
        k = _unit(gs, np.ones(1))
        assert_close(conv.bias.grad[cos] * k, gb * k, positions, what + " grad_bias")
        del rec["x"], rec["out"], rec["g_out"]


def test_full_size_stack_runs_and_is_deterministic():
    """BASELINE config 5: ten layers, 3 -> 256 channels, 4 x 4 kernels, ReLU, frequency
    max-pool 2 after layers 3, 6 and 9, batch 32, up to 780 frames x 41 bins, seed 4."""
    p = ConvStackParams(layers=10, mellin=True, kernel_time=4, kernel_freq=4, initial_channels=32,
                        factor_schedule=3, channel_factor=2, time_factor=1, freq_factor=1, in_channels=3,
                        freq_pool_after=(3, 6, 9), seed=4)
    stack = ConvStack(780, 41, p).cuda()
    assert [lay["out_channels"] for lay in stack.plan] == [32, 32, 64, 64, 64, 128, 128, 128, 256, 256]
    assert stack.out_size == (780, 5)
    gen = torch.Generator().manual_seed(4)
    lens = torch.randint(100, 781, (32,), generator=gen)
    x = torch.randn(32, 3, 780, 41, generator=gen)
    x = x * (torch.arange(780)[None, :] < lens[:, None])[:, None, :, None]     # zero past each length
    results = []
    for _ in range(2):
        for q in stack.parameters():
            q.grad = None
        xg = x.cuda().requires_grad_(True)
        out = stack(xg)
        assert tuple(out.shape) == (32, 256, 780, 5)
        loss = out.square().mean()
        loss.backward()
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(xg.grad).all())
        results.append((out.detach().clone(), xg.grad.clone(),
                        [q.grad.clone() for q in stack.parameters()]))
    assert torch.equal(results[0][0], results[1][0])
    assert torch.equal(results[0][1], results[1][1])
    for a, b in zip(results[0][2], results[1][2]):
        assert bool(torch.isfinite(a).all())
        assert torch.equal(a, b)


# ---- the non-linearity applied by the convolution kernel itself ---------------------
RELU_CASES = [
    # op, input shape, weight shape, kwargs
    ("mcorrlcorr", (3, 3, 60, 20), (40, 3, 5, 3), dict(s=(1, 1), d=(2, 1), p=(1, 1), r=(2, 0))),
    ("lcorrlcorr", (2, 3, 70, 41), (64, 3, 8, 4), dict()),
    ("lcorrlcorr", (2, 40, 30, 12), (70, 40, 3, 3), dict(d=(2, 1), p=(2, 1), r=(2, 1))),   # several channel chunks
    ("mcorr1d", (4, 6, 80), (9, 6, 7), dict(p=2)),
    ("lcorr1d", (4, 6, 80), (33, 6, 7), dict(s=2)),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16], ids=["f32", "f64", "f16"])
@pytest.mark.parametrize("case", RELU_CASES, ids=[c[0] + str(i) for i, c in enumerate(RELU_CASES)])
def test_fused_relu_equals_relu_of_the_plain_op(case, dtype):
    name, xs, ws, kw = case
    op = getattr(mconv, name)
    torch.manual_seed(RELU_CASES.index(case))
    x = torch.randn(*xs, device="cuda", dtype=dtype)
    w = torch.randn(*ws, device="cuda", dtype=dtype) / float(np.prod(ws[1:])) ** 0.5
    b = torch.randn(ws[0], device="cuda", dtype=dtype) * 0.1
    xa, wa, ba = (t.clone().requires_grad_(True) for t in (x, w, b))
    xb, wb, bb = (t.clone().requires_grad_(True) for t in (x, w, b))
    ya = op(xa, wa, ba, activation="relu", **kw)
    yb = torch.relu(op(xb, wb, bb, **kw))
    assert torch.equal(ya, yb)                             # same kernel, same sums: bit for bit
    assert float((ya == 0).float().mean()) > 0.2           # the clamp is exercised
    g = torch.randn_like(ya)
    ya.backward(g)
    yb.backward(g)
    for a, b_ in ((xa, xb), (wa, wb), (ba, bb)):
        assert torch.equal(a.grad, b_.grad)
    with pytest.raises(RuntimeError, match="activation must be None"):
        op(x, w, b, activation="tanh", **kw)


def test_windows_make_utterances_independent_of_their_batch():
    """The reference's padding-invariance check (tests/test_models.py:101-152) at the level of
    the convolution stack: the windows of an utterance give the same features whether the
    utterance is processed alone or inside a zero-padded batch."""
    from conv_stack import pack_windows
    torch.manual_seed(7)
    n, t_max, f, w_size, w_stride = 4, 50, 12, 10, 3
    lens = torch.tensor([50, 17, 33, 8])
    x = torch.randn(n, t_max, f, device="cuda")
    for i in range(n):
        x[i, lens[i]:] = 0
    params = ConvStackParams(layers=3, mellin=True, kernel_time=3, kernel_freq=3, initial_channels=8, seed=5)
    stack = ConvStack(w_size, f, params).cuda()
    windows, packed = pack_windows(x, lens, w_size, w_stride)
    lens_ = (lens - 1) // w_stride + 1
    assert windows.shape == (int(lens_.sum()), 1, w_size, f)
    together = stack(windows)
    feats = torch.nn.utils.rnn.pad_packed_sequence(
        torch.nn.utils.rnn.PackedSequence(together.sum(2).flatten(1), packed.batch_sizes,
                                          packed.sorted_indices, packed.unsorted_indices), batch_first=True)[0]
    for i in range(n):
        alone, _ = pack_windows(x[i:i + 1, :lens[i]], lens[i:i + 1], w_size, w_stride)
        ya = stack(alone).sum(2).flatten(1)
        assert ya.shape[0] == int(lens_[i])
        np.testing.assert_allclose(to_np(feats[i, :lens_[i]]), to_np(ya), rtol=1e-5, atol=1e-5)
