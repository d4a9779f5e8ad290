#!/usr/bin/env python3
"""Compile libmellin_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python cnn-mellin_amd/build.py [--force]

Sources: csrc/*.hip; output: lib/libmellin_hip.so next to this file.  Packed
FP32 VALU instructions are disabled for all device code.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "lib", "libmellin_hip.so")
ARCH = "gfx950"

FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def up_to_date():
    if not os.path.isfile(OUT):
        return False
    deps = sources() + glob.glob(os.path.join(CSRC, "*.hpp")) + \
        glob.glob(os.path.join(HERE, "..", "include", "*.h")) + [os.path.abspath(__file__)]
    return all(os.path.getmtime(d) <= os.path.getmtime(OUT) for d in deps)


def build(force=True, verbose=True):
    if not force and up_to_date():
        return OUT
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    objdir = os.path.join(HERE, "lib", "obj")
    os.makedirs(objdir, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    procs = []
    objs = []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [hipcc] + FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for src, pr in procs:
        out = pr.communicate()[0].decode()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l or "error" in l)
        if out.strip() and verbose:
            print(out)
        if pr.returncode != 0:
            print(out)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-fno-gpu-rdc"] + objs + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build(force="--force" in sys.argv or True)
    print("built", OUT)
