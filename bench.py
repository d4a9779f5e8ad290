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
the longest (median of at least 100 launches, each timed with HIP events on the
launch stream), against the roof that binds it: the time its algorithmic bytes
need at the HBM peak against the time its matrix instructions need at their
peak (bf16 instructions, six per fp32 product, when the kernels ran in the
library's default bf16x3 mode; fp32 instructions otherwise), with the other
figure alongside.  `cpu_baseline` times the CPU checker on the same batch on
the host cores.

Before the clock starts the step is repeated until the GPU has been busy for
50 ms (`prewarm_ms`; outside the timed region, on top of --warmup): a step
takes a quarter of a millisecond and a chip that has idled runs its first few
milliseconds 5-10 % slow.
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
BF16_PEAK_TFLOPS = 2500.0    # MI355X dense bf16 matrix (MFMA), published
PREWARM_MS = 50.0
MIN_PASS_REPS = 100

# HBM bytes per launch of each pass at this workload come from the data file that is written
# together with the profile summary of the same name under profiles/ (rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE per dispatch, scaled by what the same counters read for a plain
# 256 MiB device copy).  An entry is used only if the pass ran the variant and the math mode
# that were profiled.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_cfg3_hbm_bytes.json")


def measured_traffic(pass_name, variant, math):
    try:
        with open(TRAFFIC_FILE) as f:
            e = json.load(f)["passes"][pass_name]
    except (OSError, KeyError, ValueError):
        return None
    return e["bytes"] if (e.get("variant"), e.get("math")) == (variant, math) else None


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
        nbytes = hip.lib.mellin_corr2d_forward_workspace(kind_x, 4, *self.dims)
        self.ws_fwd = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        self.ws_fwd_bytes = nbytes
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
        hip.corr2d_forward(self.kind_x, self.x, self.w, self.b, self.out, self.dims,
                           workspace=self.ws_fwd, workspace_bytes=self.ws_fwd_bytes)

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
    """Median duration of one call, in microseconds: every call sits between two HIP events
    on the launch stream (torch's current stream is the stream the library launches on)."""
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    marks[0].record()
    for i in range(reps):
        fn()
        marks[i + 1].record()
    marks[-1].synchronize()
    times = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(reps))
    return times[len(times) // 2]


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
    extra = {}
    if oracle.have_ref():
        # the reference's own header (compiled from the reference checkout where one was present
        # at build time) has the Mellin x linear kernels only: the same half of the step through
        # it and through the port, to show that the port is not the slower of the two
        L = layers[0]
        x = np.ascontiguousarray(L.x_cpu.numpy()[:slice_n])
        go = np.ascontiguousarray(L.go_cpu.numpy()[:slice_n])
        w, b = L.w_cpu.numpy(), L.b_cpu.numpy()
        for impl in ("ref", "port"):
            ts = []
            for _ in range(5):
                t0 = time.perf_counter()
                oracle.mcorrlcorr(x, w, b, 1, 1, 0, 1, 0, impl=impl)
                oracle.mcorrlcorr_backward(x, w, go, 1, 1, 0, 1, impl=impl)
                ts.append(time.perf_counter() - t0)
            extra["mconv2d_half_%s_ms" % ("reference" if impl == "ref" else "port")] = round(sorted(ts)[2] * 1e3, 2)
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": min(threads, cores),
            "kind": "port", **extra,
            "sample": "same step on utterances 0..%d of 32 (%.0f MB algorithmic), median of %d repetitions "
                      "(%.1f s of CPU work in all), %.2f s each; %.0f frames/s"
                      % (slice_n - 1, nbytes / 1e6, reps, sum(times), med, slice_n * CFG["ngx"] / med),
            "frames_per_s": round(slice_n * CFG["ngx"] / med, 1)}


def other_math_leg(args, dev, torch, hip, steps=30, reps=30):
    """The same step once more under the other math mode (outside the main timed region):
    wall-clock per step over `steps` steps after 10 warm-up steps, and per-pass medians."""
    other = hip.MATH_FP32 if args.math == "bf16x3" else hip.MATH_BF16X3
    hip.set_math(other)
    try:
        gen = torch.Generator().manual_seed(2)
        layers = [Layer(hip.AX_MCORR, "mconv2d", gen, dev), Layer(hip.AX_LCORR, "lconv2d", gen, dev)]   # (workspaces of this mode)

        def step():
            for L in layers:
                L.forward()
                L.backward_input()
                L.backward_weight()
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        per_pass, maths = {}, {}
        for L in layers:
            for pname, fn in L.passes():
                key = "%s.%s" % (L.name, pname)
                per_pass[key] = round(time_pass(fn, reps, torch), 2)
                maths[key] = "bf16x3" if hip.last_math() == hip.MATH_BF16X3 else "fp32"
        return {"ms_per_step": round(ms, 4), "steps": steps, "per_pass_us": per_pass, "per_pass_math": maths}
    finally:
        hip.set_math(hip.MATH_BF16X3 if args.math == "bf16x3" else hip.MATH_FP32)


def other_configs(torch, reps=20):
    """Per-pass times of BASELINE configuration 4 (wide layer, linear and Mellin x axis) and
    forward + backward of the two 10-layer stacks of configuration 5, by time_layers.py's own
    routines, `reps` timed calls each (outside the main timed region; not bench lines)."""
    import time_layers
    out = {"reps": reps, "cfg4": {}, "cfg5_stack_forward_backward_ms": {}}

    def keep_layer(rec):
        out["cfg4"][rec["layer"].split()[-1]] = {k: rec[k]["us"] for k in ("forward", "grad_input", "grad_weight")}

    def keep_stack(rec):
        if "stack" in rec:
            out["cfg5_stack_forward_backward_ms"][rec["stack"]] = rec["forward_backward_ms"]
    time_layers.run_cfg4(reps, torch.float32, emit=keep_layer)
    time_layers.run_stack(reps, torch.float32, emit=keep_stack, per_layer=False)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--math", choices=["bf16x3", "fp32"], default="bf16x3",
                    help="how the matrix kernels form fp32 products (library default: bf16x3)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the legs outside the timed region: the same step under the fp32 math mode and the "
                         "other configurations (wide layer, 10-layer stacks)")
    ap.add_argument("--variant", default=None, help="force a kernel variant (e.g. generic)")
    ap.add_argument("--cpu-slice", type=int, default=32, help="utterances in the CPU baseline sample")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain device copy of known size (to scale profiler byte counters)")
    ap.add_argument("--only-pass", default=None, metavar="LAYER.PASS",
                    help="only launch one pass --launches times, e.g. lconv2d.grad_input (for profiler "
                         "runs: every kernel in the trace then belongs to that pass)")
    ap.add_argument("--launches", type=int, default=10)
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
    hip.set_math(hip.MATH_BF16X3 if args.math == "bf16x3" else hip.MATH_FP32)
    gen = torch.Generator().manual_seed(2)
    layers = [Layer(hip.AX_MCORR, "mconv2d", gen, dev), Layer(hip.AX_LCORR, "lconv2d", gen, dev)]

    if args.only_pass:
        fns = {"%s.%s" % (L.name, pname): fn for L in layers for pname, fn in L.passes()}
        if args.only_pass not in fns:
            sys.exit("--only-pass: one of %s" % ", ".join(fns))
        for _ in range(args.launches):
            fns[args.only_pass]()
        torch.cuda.synchronize()
        print(json.dumps({"pass": args.only_pass, "launches": args.launches, "variant": hip.last_variant(),
                          "math": "bf16x3" if hip.last_math() == hip.MATH_BF16X3 else "fp32"}))
        return

    def step():
        for L in layers:
            L.forward()
            L.backward_input()
            L.backward_weight()

    # pre-warm: steps until the GPU has worked for PREWARM_MS (disclosed, outside the timed region)
    pre0, pre1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    pre0.record()
    prewarm_ms, prewarm_steps = 0.0, 0
    while prewarm_ms < PREWARM_MS:
        for _ in range(20):
            step()
        prewarm_steps += 20
        pre1.record()
        pre1.synchronize()
        prewarm_ms = pre0.elapsed_time(pre1)
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
    per_pass, variants, maths = {}, {}, {}
    for L in layers:
        for pname, fn in L.passes():
            key = "%s.%s" % (L.name, pname)
            per_pass[key] = time_pass(fn, max(MIN_PASS_REPS, args.steps), torch)
            variants[key] = hip.last_variant()
            maths[key] = "bf16x3" if hip.last_math() == hip.MATH_BF16X3 else "fp32"
    dom = max(per_pass, key=per_pass.get)
    domL = layers[0] if dom.startswith("mconv2d") else layers[1]
    dom_us = per_pass[dom]
    achieved_gbs = domL.bytes_per_pass / dom_us / 1e3
    dom_tflops = 2 * domL.macs_per_pass / dom_us / 1e6
    # which roof: the time the algorithmic bytes need at the HBM peak against the time the
    # matrix instructions need at theirs (six bf16 instructions' worth per fp32 product in
    # bf16x3 mode, where every fp32 operand is the exact sum of three bf16 parts)
    flops = 2 * domL.macs_per_pass
    if maths[dom] == "bf16x3":
        matrix_flops, matrix_peak, matrix_unit = 6 * flops, BF16_PEAK_TFLOPS, "bf16"
    else:
        matrix_flops, matrix_peak, matrix_unit = flops, FP32_PEAK_TFLOPS, "fp32"
    t_hbm_us = domL.bytes_per_pass / HBM_PEAK_GBS / 1e3
    t_matrix_us = matrix_flops / matrix_peak / 1e6
    matrix_tflops = matrix_flops / dom_us / 1e6
    traffic = measured_traffic(dom, variants[dom], maths[dom])
    if t_matrix_us > t_hbm_us:
        roof = {"bound": "mfma", "achieved": round(matrix_tflops, 2), "peak": matrix_peak, "unit": "TFLOP/s",
                "frac": round(matrix_tflops / matrix_peak, 4)}
    else:
        roof = {"bound": "hbm", "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved_gbs / HBM_PEAK_GBS, 4)}
    roof.update({"traffic": traffic, "kernel": dom, "variant": variants[dom], "math": maths[dom],
                 "median_us": round(dom_us, 2), "reps": max(MIN_PASS_REPS, args.steps),
                 "algorithmic_bytes": domL.bytes_per_pass, "algorithmic_flops": flops,
                 "us_at_hbm_peak": round(t_hbm_us, 2), "us_at_matrix_peak": round(t_matrix_us, 2),
                 "matrix_instructions": matrix_unit, "matrix_flops_executed": matrix_flops,
                 "hbm_GBps": round(achieved_gbs, 1), "hbm_frac": round(achieved_gbs / HBM_PEAK_GBS, 4),
                 "matrix_TFLOPs": round(matrix_tflops, 2), "matrix_frac": round(matrix_tflops / matrix_peak, 4),
                 "fp32_equivalent_TFLOPs": round(dom_tflops, 2)})

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
                   "GFLOP_per_step": round(step_flops / 1e9, 3),
                   "arithmetic": ("fp32 storage, fp32 accumulation; products of the matrix kernels: every fp32 "
                                  "operand as the exact sum of three bf16 parts (rounded to nearest), the six "
                                  "largest of the nine cross products on the bf16 matrix cores (what is dropped "
                                  "is at most 1.01 * 2^-23 of a product, worst case)" if args.math == "bf16x3" else
                                  "fp32 storage, accumulation and matrix instructions")},
        "prewarm_ms": round(prewarm_ms, 1), "prewarm_steps": prewarm_steps,
        "frames_per_s": round(frames / (elapsed / args.steps), 1),
        "pct_hbm_roofline": round(100.0 * step_bytes / (elapsed / args.steps) / 1e9 / HBM_PEAK_GBS, 2),
        "tflops": round(step_flops / (elapsed / args.steps) / 1e12, 2),
        "roofline": roof,
        "per_pass_us": {k: round(v, 2) for k, v in per_pass.items()},
        "per_pass_variant": variants,
        "per_pass_math": maths,
    }
    line["per_pass_roofline"] = {
        k: {"hbm_frac": round((layers[0] if k.startswith("mconv2d") else layers[1]).bytes_per_pass / v / 1e3
                              / HBM_PEAK_GBS, 4),
            "fp32_equivalent_TFLOPs": round(2 * (layers[0] if k.startswith("mconv2d") else layers[1]).macs_per_pass
                                            / v / 1e6, 2)}
        for k, v in per_pass.items()}
    if not args.no_extras:
        line["fp32_math" if args.math == "bf16x3" else "bf16x3_math"] = other_math_leg(args, dev, torch, hip)
        line["other_configs"] = other_configs(torch)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(layers, args.cpu_slice)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
