"""Builds the HIP library (libtensornet_amd.so) in-tree with hipcc for gfx950.

    python -m tensornet_amd.build

hipcc cross-compiles without a GPU.  The flags keep fp32 arithmetic IEEE
(no FMA contraction, correctly rounded divide / sqrt) so that optimizer
updates can be compared element for element with a CPU evaluation, and turn
packed-fp32 instruction selection off.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtensornet_amd.so")
SOURCES = ["core.hip", "dense_table.hip", "sparse_table.hip"]
HEADERS = ["tn_common.h", "sparse_kernels.h"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
