"""Builds libswitchyard_moe.so (the gfx950 kernels and their C ABI) in-tree with hipcc.

    python -m switchyard_amd.build

The library has no torch, pybind or Python dependency, so it cross-compiles on a machine
without a GPU. The counterpart of the reference's JIT build (switchyard/kernels.py:12-20)."""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libswitchyard_moe.so")
SOURCES = ["abi.hip", "route.hip", "sort.hip", "front.hip", "combine.hip", "gemv.hip", "gemm.hip", "decode.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # hipcc -O3 must not form packed fp32 instructions from scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    return os.environ.get("HIPCC") or os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")


def build(verbose=False, extra=()):
    """Compile every source into one shared library; raises on failure."""
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc(), *[f for f in FLAGS if f != "-shared"], *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        objs.append(obj)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
    print(LIB)
