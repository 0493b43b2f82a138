"""Builds libnsa_hip.so (all HIP kernels + the C ABI) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnsa_hip.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # never let the compiler form packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results in ordinary vector registers: the walks' accumulators feed VALU code (softmax, scaling, stores), and from
    # accumulation registers every element would first need a copy instruction (a sixth of the forward walk's VALU work)
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


def build(verbose: bool = False) -> str:
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not srcs:
        raise RuntimeError("no HIP sources found under " + CSRC)
    cmd = ["hipcc", *FLAGS, *srcs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
