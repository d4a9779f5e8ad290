#!/usr/bin/env python3
"""Per-pass timings on one MI355X of the layer shapes beside the benchmark's own.

    python time_layers.py cfg3            # the benchmark's own layer, linear and Mellin x axis
    python time_layers.py cfg4            # wide 2-D layer, linear and Mellin x axis
    python time_layers.py cfg2            # 1-D layers over the (s, d, p) grid
    python time_layers.py stack           # the 10-layer 3 -> 256 stacks, layer by layer
    python time_layers.py cfg4 --dtype half   # the same on half-precision tensors (the stack: under autocast)

Every pass is one call of the C ABI on pre-allocated tensors, timed with HIP events
on the launch stream.  One JSON object per line: the layer, its output extent, and
for forward / grad_input / grad_weight the microseconds, the kernel variant that ran
and fp32 TFLOP/s from the exact multiply-accumulate count (pairs of output position
and filter tap that land inside the input, per axis).  Needs the HIP library and a GPU.
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "cnn-mellin_amd"))


def tap_pairs(kind, nf, ng, nh, s, d, p, u=1):
    """(output position, filter tap) pairs of one axis whose source lies in the input."""
    import _mellin_hip as hip
    pairs = 0
    for h in range(nh):
        for f in range(nf):
            if kind == hip.AX_MCORR:
                num, den, off = (h + s) * (f + d), p + 1, u
            else:
                num, den, off = s * h + d * f - p, u, 0
            pairs += num % den == 0 and 0 <= num // den - off < ng
    return pairs


def event_us(fn, reps):
    import torch
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) * 1e3 / reps


def time_layer(tag, kind_x, x, w, b, s, d, p, r, reps, activation=None):
    """x (N, C_in, T, F), w (C_out, C_in, kx, ky) on the GPU; returns the record and the output."""
    import torch
    import mconv
    import _mellin_hip as hip
    op = mconv._ext_mcorrlcorr if kind_x == hip.AX_MCORR else mconv._ext_lcorrlcorr
    out = op(x, w, b, s, d, p, (1, 1), r)
    n, c_in, ng = x.shape[0], x.shape[1], tuple(x.shape[2:])
    c_out, nf, nh = w.shape[0], tuple(w.shape[2:]), tuple(out.shape[2:])
    dims = hip._dims(n, c_in, c_out, nf, ng, nh, s, d, p, (1, 1))
    go = torch.randn_like(out)
    o2, gi, gw = torch.empty_like(out), torch.empty_like(x), torch.empty_like(w)
    macs = (n * c_out * c_in * tap_pairs(kind_x, nf[0], ng[0], nh[0], s[0], d[0], p[0]) *
            tap_pairs(hip.AX_LCORR, nf[1], ng[1], nh[1], s[1], d[1], p[1]))
    rec = {"layer": tag, "in": [c_in, *ng], "out": [c_out, *nh], "gmac": round(macs / 1e9, 3)}
    for name, fn in (("forward", lambda: hip.corr2d_forward(kind_x, x, w, b, o2, dims)),
                     ("grad_input", lambda: hip.corr2d_backward_input(kind_x, w, go, gi, dims)),
                     ("grad_weight", lambda: hip.corr2d_backward_weight(kind_x, x, go, gw, dims))):
        us = event_us(fn, reps)
        rec[name] = {"us": round(us, 1), "variant": hip.last_variant(),
                     "math": {hip.MATH_BF16X3: "bf16x3", hip.MATH_F16: "f16"}.get(hip.last_math(), "fp32"),
                     "tflops": round(2 * macs / us / 1e6, 1)}
    return rec, out


def run_cfg3(reps, dtype):
    import torch
    import _mellin_hip as hip
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(32, 3, 512, 41, device="cuda", generator=gen).to(dtype)
    bound = (3 * 32) ** -0.5
    w = ((torch.rand(64, 3, 8, 4, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(64, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    for kind, name in ((hip.AX_LCORR, "lconv2d"), (hip.AX_MCORR, "mconv2d")):
        rec, _ = time_layer("cfg3 " + name, kind, x, w, b, (1, 1), (1, 1), (0, 0), (0, 0), reps)
        print(json.dumps(rec), flush=True)


def _emit(rec):
    print(json.dumps(rec), flush=True)


def run_cfg4(reps, dtype, emit=_emit):
    import torch
    import _mellin_hip as hip
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(32, 128, 256, 41, device="cuda", generator=gen).to(dtype)
    bound = (128 * 9) ** -0.5
    w = ((torch.rand(256, 128, 3, 3, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(256, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    for kind, name in ((hip.AX_LCORR, "lconv2d"), (hip.AX_MCORR, "mconv2d")):
        rec, _ = time_layer("cfg4 " + name, kind, x, w, b, (1, 1), (2, 1), (2, 1), (2, 1), reps)
        emit(rec)


def run_cfg2(reps, dtype):
    import torch
    import _mellin_hip as hip
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(32, 41, 780, 1, device="cuda", generator=gen).to(dtype)
    bound = (41 * 8) ** -0.5
    w = ((torch.rand(128, 41, 8, 1, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    b = ((torch.rand(128, device="cuda", generator=gen) * 2 - 1) * bound).to(dtype)
    for s in (1, 2):
        for d in (1, 2):
            for p in (0, 3):
                for kind, name in ((hip.AX_MCORR, "mcorr1d"), (hip.AX_LCORR, "lcorr1d")):
                    rec, _ = time_layer("cfg2 %s s=%d d=%d p=%d" % (name, s, d, p), kind, x, w, b,
                                        (s, 1), (d, 1), (p, 0), (0, 0), reps)
                    print(json.dumps(rec), flush=True)


def run_stack(reps, dtype, emit=_emit, per_layer=True):
    import time
    import torch
    import _mellin_hip as hip
    from conv_stack import ConvStack, ConvStackParams, FrameClassifier
    for mellin in (True, False):
        params = ConvStackParams(layers=10, mellin=mellin, kernel_time=4, kernel_freq=4, initial_channels=32,
                                 factor_schedule=3, channel_factor=2, time_factor=1, freq_factor=1,
                                 in_channels=3, freq_pool_after=(3, 6, 9), seed=4)
        model = FrameClassifier(ConvStack(780, 41, params), 62).cuda()
        stack = model.stack
        x = torch.randn(32, 3, 780, 41, device="cuda", requires_grad=True)

        def step():
            # the conv stack and its Linear -> 62 log-softmax head, summed over frames
            # (half: fp32 parameters, the layers cast their operands under autocast)
            with torch.autocast("cuda", enabled=dtype == torch.float16):
                loss = model(x).float().square().mean()
            loss.backward()
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            step()
        torch.cuda.synchronize()
        name = "mellin" if mellin else "linear"
        emit({"stack": name, "forward_backward_ms": round((time.perf_counter() - t0) / reps * 1e3, 2)})
        if not per_layer:
            continue
        h = x.detach().to(dtype)
        for no, (lay, conv) in enumerate(zip(stack.plan, stack.convs), 1):
            kind = hip.AX_MCORR if lay["kind"] == "mcorrlcorr" else hip.AX_LCORR
            rec, out = time_layer("%s stack layer %d" % (name, no), kind, h, conv.weight.detach().to(dtype),
                                  conv.bias.detach().to(dtype) if conv.bias is not None else None,
                                  lay["s"], lay["d"], lay["p"], lay["r"], reps)
            emit(rec)
            h = torch.relu(out)
            if lay["pool"]:
                h = torch.nn.functional.max_pool2d(h, (1, 2))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("config", choices=["cfg2", "cfg3", "cfg4", "stack"])
    ap.add_argument("--reps", type=int, default=10, help="timed calls per pass")
    ap.add_argument("--math", choices=["bf16x3", "fp32"], default="bf16x3",
                    help="how the matrix kernels form fp32 products (library default: bf16x3)")
    ap.add_argument("--dtype", choices=["float32", "half"], default="float32",
                    help="half: half-precision tensors through the f16 entry points")
    ap.add_argument("--variant", default=None,
                    help="a kernel variant for comparisons (mellin_set_variant: two-pass, one-launch, classes, "
                         "class-launches, widen, generic)")
    args = ap.parse_args()
    import torch
    if not torch.cuda.is_available():
        sys.exit("time_layers.py needs a GPU")
    torch.cuda.set_device(0)
    import _mellin_hip as hip
    hip.set_math(hip.MATH_BF16X3 if args.math == "bf16x3" else hip.MATH_FP32)
    hip.set_variant(args.variant)
    dtype = torch.float16 if args.dtype == "half" else torch.float32
    {"cfg2": run_cfg2, "cfg3": run_cfg3, "cfg4": run_cfg4, "stack": run_stack}[args.config](args.reps, dtype)


if __name__ == "__main__":
    main()
