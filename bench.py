#!/usr/bin/env python3
"""Throughput of the Mellin / linear correlation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = forward, input-gradient and weight-gradient of a Mellin x linear
layer ("mconv2d") AND of a linear x linear layer ("lconv2d") over one
fbank-shaped synthetic batch: x (32, 3, 512, 41), weight (64, 3, 8, 4),
s = d = u = 1, p = 0, fp32, inputs resident in HBM before the clock starts.
Prints one JSON line.  `value` is algorithmic GB/s (each operand read once,
each result written once) over the whole step; `frames_per_s` counts the
32 x 512 input frames once per step.  `roofline` describes the pass that takes
the longest, timed with HIP events on the launch stream: against the fp32
matrix peak when its arithmetic intensity (algorithmic FLOP per algorithmic
byte) is above the machine's ridge point, against the HBM peak otherwise, with
the other figure alongside.  `cpu_baseline` times the CPU checker on the same
batch on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "cnn-mellin_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3     # MI355X fp32 matrix (MFMA) = packed vector fp32, published

# HBM bytes per launch of each pass at this workload, measured with
#   rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --steps 3 --warmup 1 --no-cpu
#   rocprofv3 --pmc WRITE_SIZE -- python3 bench.py --steps 3 --warmup 1 --no-cpu
# (KiB per dispatch, summed over the kernels of the pass) and scaled by what the same
# counters read for a plain 256 MiB device copy (--copy-calibration): FETCH_SIZE x 2.0,
# WRITE_SIZE x 1.0.  The summary is kept under profiles/.
MEASURED_TRAFFIC_BYTES = {
    "mconv2d.forward": 35.3e6, "mconv2d.grad_input": 88.3e6, "mconv2d.grad_weight": 47.8e6,
    "lconv2d.forward": 195.6e6, "lconv2d.grad_input": 190.1e6, "lconv2d.grad_weight": 214.3e6,
}
MEASURED_TRAFFIC_VARIANTS = {
    "mconv2d.forward": "mfma", "mconv2d.grad_input": "mfma-taps+fold", "mconv2d.grad_weight": "mfma-rows",
    "lconv2d.forward": "mfma", "lconv2d.grad_input": "mfma-fused", "lconv2d.grad_weight": "mfma-rows",
}

CFG = dict(batch=32, c_in=3, c_out=64, ngx=512, ngy=41, nfx=8, nfy=4,
           s=(1, 1), d=(1, 1), p=(0, 0), u=(1, 1))


def layer_shapes(kind_x):
    import mconv
    import _mellin_hip as hip
    c = CFG
    valid_x = mconv.mcorr_valid_size if kind_x == hip.AX_MCORR else mconv.lcorr_valid_size
    nhx = valid_x(c["nfx"], c["ngx"])
    nhy = mconv.lcorr_valid_size(c["nfy"], c["ngy"])
    return nhx, nhy


def pass_bytes_flops(nhx, nhy):
    c = CFG
    x = c["batch"] * c["c_in"] * c["ngx"] * c["ngy"] * 4
    w = c["c_out"] * c["c_in"] * c["nfx"] * c["nfy"] * 4
    o = c["batch"] * c["c_out"] * nhx * nhy * 4
    return x + w + o


def count_macs(kind_x, nhx, nhy):
    """Exact multiply-accumulate count of one pass from the tap predicate."""
    import _mellin_hip as hip
    c = CFG
    px = 0
    for hx in range(nhx):
        for fx in range(c["nfx"]):
            gx = (hx + 1) * (fx + 1) - 1 if kind_x == hip.AX_MCORR else hx + fx
            px += 0 <= gx < c["ngx"]
    py = sum(0 <= hy + fy < c["ngy"] for hy in range(nhy) for fy in range(c["nfy"]))
    return c["batch"] * c["c_out"] * c["c_in"] * px * py


class Layer:
    """Pre-allocated operands of one layer type; every pass is one C-ABI call."""

    def __init__(self, kind_x, name, gen, dev):
        import torch
        import _mellin_hip as hip
        c = CFG
        self.kind_x, self.name = kind_x, name
        self.nhx, self.nhy = layer_shapes(kind_x)
        self.dims = hip._dims(c["batch"], c["c_in"], c["c_out"], (c["nfx"], c["nfy"]),
                              (c["ngx"], c["ngy"]), (self.nhx, self.nhy), c["s"], c["d"], c["p"], c["u"])
        bound = (c["c_in"] * c["nfx"] * c["nfy"]) ** -0.5
        self.x_cpu = torch.randn(c["batch"], c["c_in"], c["ngx"], c["ngy"], generator=gen)
        self.w_cpu = (torch.rand(c["c_out"], c["c_in"], c["nfx"], c["nfy"], generator=gen) * 2 - 1) * bound
        self.b_cpu = (torch.rand(c["c_out"], generator=gen) * 2 - 1) * bound
        self.go_cpu = torch.randn(c["batch"], c["c_out"], self.nhx, self.nhy, generator=gen)
        self.x, self.w, self.b, self.go = (t.to(dev) for t in (self.x_cpu, self.w_cpu, self.b_cpu, self.go_cpu))
        self.out = torch.empty_like(self.go)
        self.gi = torch.empty_like(self.x)
        self.gw = torch.empty_like(self.w)
        nbytes = hip.lib.mellin_corr2d_backward_weight_workspace(kind_x, 4, *self.dims)
        self.ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        self.ws_bytes = nbytes
        nbytes = hip.lib.mellin_corr2d_backward_input_workspace(kind_x, 4, *self.dims)
        self.ws_in = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        self.ws_in_bytes = nbytes
        self.bytes_per_pass = pass_bytes_flops(self.nhx, self.nhy)
        self.macs_per_pass = count_macs(kind_x, self.nhx, self.nhy)

    def forward(self):
        import _mellin_hip as hip
        hip.corr2d_forward(self.kind_x, self.x, self.w, self.b, self.out, self.dims)

    def backward_input(self):
        import _mellin_hip as hip
        hip.corr2d_backward_input(self.kind_x, self.w, self.go, self.gi, self.dims,
                                  workspace=self.ws_in, workspace_bytes=self.ws_in_bytes)

    def backward_weight(self):
        import _mellin_hip as hip
        hip.corr2d_backward_weight(self.kind_x, self.x, self.go, self.gw, self.dims,
                                   workspace=self.ws, workspace_bytes=self.ws_bytes)

    def passes(self):
        return [("forward", self.forward), ("grad_input", self.backward_input),
                ("grad_weight", self.backward_weight)]


def time_pass(fn, reps, torch):
    """Average duration of one call, in microseconds, from HIP events on the launch stream."""
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


def cpu_baseline(layers, slice_n, reps=25):
    """The CPU checker (restatement of the reference's OpenMP kernels) on the first
    `slice_n` utterances of the same batch: forward + both gradients of both layers."""
    import numpy as np
    from oracle import oracle
    cores = len(os.sched_getaffinity(0))
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        for L in layers:
            fwd = oracle.mcorrlcorr if L.name == "mconv2d" else oracle.lcorrlcorr
            bwd = oracle.mcorrlcorr_backward if L.name == "mconv2d" else oracle.lcorrlcorr_backward
            x = np.ascontiguousarray(L.x_cpu.numpy()[:slice_n])
            w, b = L.w_cpu.numpy(), L.b_cpu.numpy()
            go = np.ascontiguousarray(L.go_cpu.numpy()[:slice_n])
            fwd(x, w, b, 1, 1, 0, 1, 0)
            bwd(x, w, go, 1, 1, 0, 1)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    nbytes = sum(3 * (L.bytes_per_pass - L.w.numel() * 4) * slice_n / CFG["batch"] + 3 * L.w.numel() * 4
                 for L in layers)
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": min(threads, cores),
            "kind": "port",
            "sample": "same step on utterances 0..%d of 32 (%.0f MB algorithmic), median of %d repetitions "
                      "(%.1f s of CPU work in all), %.2f s each; %.0f frames/s"
                      % (slice_n - 1, nbytes / 1e6, reps, sum(times), med, slice_n * CFG["ngx"] / med),
            "frames_per_s": round(slice_n * CFG["ngx"] / med, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a step is a third of a millisecond and the first few milliseconds after an idle spell run
    # 5-8 % slow (measured: 5 warm-up steps 0.358 ms/step, 50 or more 0.335), hence the defaults
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--variant", default=None, help="force a kernel variant (e.g. generic)")
    ap.add_argument("--cpu-slice", type=int, default=32, help="utterances in the CPU baseline sample")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain device copy of known size (to scale profiler byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (got --gpus %d)" % args.gpus)

    import torch
    import _mellin_hip as hip
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        # 256 MiB read + 256 MiB written per launch, ten launches
        src = torch.randn(64 * 1024 * 1024, device=dev)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 4, "copy_bytes_written": src.numel() * 4,
                          "launches": 10}))
        return
    hip.set_variant(args.variant)
    gen = torch.Generator().manual_seed(2)
    layers = [Layer(hip.AX_MCORR, "mconv2d", gen, dev), Layer(hip.AX_LCORR, "lconv2d", gen, dev)]

    def step():
        for L in layers:
            L.forward()
            L.backward_input()
            L.backward_weight()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    step_bytes = sum(3 * L.bytes_per_pass for L in layers)
    step_flops = sum(3 * 2 * L.macs_per_pass for L in layers)
    frames = CFG["batch"] * CFG["ngx"]

    # per-pass durations (one kernel chain per pass) for the roofline of the dominant one
    per_pass = {}
    variants = {}
    for L in layers:
        for pname, fn in L.passes():
            per_pass["%s.%s" % (L.name, pname)] = time_pass(fn, max(10, args.steps), torch)
            variants["%s.%s" % (L.name, pname)] = hip.last_variant()
    dom = max(per_pass, key=per_pass.get)
    domL = layers[0] if dom.startswith("mconv2d") else layers[1]
    dom_us = per_pass[dom]
    achieved_gbs = domL.bytes_per_pass / dom_us / 1e3
    dom_tflops = 2 * domL.macs_per_pass / dom_us / 1e6
    # which roof: arithmetic intensity against the ridge point of the two peaks
    intensity = 2 * domL.macs_per_pass / domL.bytes_per_pass
    ridge = FP32_PEAK_TFLOPS * 1e3 / HBM_PEAK_GBS
    traffic = MEASURED_TRAFFIC_BYTES.get(dom) if variants[dom] == MEASURED_TRAFFIC_VARIANTS.get(dom) else None
    if intensity > ridge:
        roof = {"bound": "mfma", "achieved": round(dom_tflops, 2), "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(dom_tflops / FP32_PEAK_TFLOPS, 4)}
    else:
        roof = {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved_gbs / HBM_PEAK_GBS, 4)}
    roof.update({"traffic": traffic, "kernel": dom, "variant": variants[dom], "avg_us": round(dom_us, 2),
                 "flop_per_byte": round(intensity, 1), "ridge_flop_per_byte": round(ridge, 1),
                 "algorithmic_bytes": domL.bytes_per_pass, "algorithmic_flops": 2 * domL.macs_per_pass,
                 "hbm_GBps": round(achieved_gbs, 1), "hbm_frac": round(achieved_gbs / HBM_PEAK_GBS, 4),
                 "fp32_TFLOPs": round(dom_tflops, 2), "fp32_frac": round(dom_tflops / FP32_PEAK_TFLOPS, 4)})

    line = {
        "metric": "mconv2d+lconv2d fwd+bwd GB/s and frames/sec on 1 MI355X; % HBM roofline",
        "value": round(step_bytes / elapsed * args.steps / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg3 fbank batch x(32,3,512,41) w(64,3,8,4) s=d=u=1 p=0: "
                               "mconv2d (Mellin x linear) and lconv2d (linear x linear), each forward + "
                               "input-gradient + weight-gradient",
                   "algorithmic_MB_per_step": round(step_bytes / 1e6, 3),
                   "GFLOP_per_step": round(step_flops / 1e9, 3)},
        "frames_per_s": round(frames / (elapsed / args.steps), 1),
        "pct_hbm_roofline": round(100.0 * step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS, 2),
        "tflops": round(step_flops / (elapsed / args.steps) / 1e12, 2),
        "roofline": roof,
        "per_pass_us": {k: round(v, 2) for k, v in per_pass.items()},
        "per_pass_variant": variants,
    }
    line["per_pass_roofline"] = {
        k: {"hbm_frac": round((layers[0] if k.startswith("mconv2d") else layers[1]).bytes_per_pass / v / 1e3
                              / HBM_PEAK_GBS, 4),
            "fp32_frac": round(2 * (layers[0] if k.startswith("mconv2d") else layers[1]).macs_per_pass / v / 1e6
                               / FP32_PEAK_TFLOPS, 4)}
        for k, v in per_pass.items()}
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(layers, args.cpu_slice)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
