"""Builds libbdh_mi355x.so (the C-ABI library) in-tree with hipcc for gfx950.

    python -m burn_dragon_amd.build

The library depends only on the HIP runtime.  It is cross-compiled: no GPU is needed.
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libbdh_mi355x.so")
SOURCES = ["bdh_api.hip", "state_step.hip", "state_deferred.hip", "projections.hip", "model.hip", "attention_parallel.hip", "prefill.hip",
           "sampling.hip", "viz_taps.hip", "model_small.hip", "model_phase.hip", "probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",  # every fused multiply-add in the kernels is an explicit fmaf
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build_library(verbose: bool = False) -> str:
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        # hipcc's host pass does not know the packed-fp32 target feature and says so: harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            failed = True
            print(f"--- {src} ---\n{out}", file=sys.stderr)
        elif verbose and out.strip():
            print(f"--- {src} ---\n{out}")
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
