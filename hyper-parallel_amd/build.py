"""Builds libhpfp8.so (HIP kernels + C ABI) in-tree with hipcc for gfx950.

Usage: python build.py [--force]
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "hpfp8", "libhpfp8.so")
SOURCES = ["capi.hip", "quantize.hip", "bucket.hip", "grouped.hip", "gemm.hip"]
HEADERS = ["hpfp8_device.h", "hpfp8_host.h", os.path.join("..", "..", "include", "hpfp8.h")]


def _flags():
    # full IEEE division/sqrt, denormals kept, no packed fp32 arithmetic
    return [
        "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
        "-fno-fast-math", "-ffp-contract=off", "-fno-gpu-flush-denormals-to-zero",
        "-fhip-fp32-correctly-rounded-divide-sqrt",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wno-unused-command-line-argument",
    ]


def needs_build() -> bool:
    if not os.path.exists(OUT):
        return True
    t = os.path.getmtime(OUT)
    deps = [os.path.join(CSRC, s) for s in SOURCES + HEADERS] + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = False) -> str:
    if not force and not needs_build():
        return OUT
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + _flags() + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
