"""Builds libapc_hip.so (HIP kernels + C ABI) in-tree for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
ROOT = os.path.dirname(PKG)
LIB = os.path.join(PKG, "libapc_hip.so")

# -ffp-contract=off: every product and sum of the cost model is rounded on its
# own, as in the Python it replaces; a fused multiply-add would change bits.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(ROOT, "include"),
]


def build(verbose: bool = True) -> str:
    srcs = [os.path.join(HERE, f) for f in ("apc.hip", "lut.hip", "score.hip", "sample.hip", "passes.hip", "schedule.hip", "nccl_plan.cpp")]
    cmd = ["hipcc"] + HIPCC_FLAGS + srcs + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
