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
SOURCES = ["core.hip", "dense_table.hip", "sparse_table.hip", "checkpoint.hip"]

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


HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "host_mirror_test.cc")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-lz", "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def build_host_test(verbose=True):
    """Builds the C++ program that drives the library through include/tensornet_amd.hpp."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-std=c++17", "-O1", "-I", os.path.join(ROOT, "include"), HOST_TEST_SRC, "-L", HERE,
           "-ltensornet_amd", "-Wl,-rpath,$ORIGIN/../../tensornet_amd", "-o", HOST_TEST_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return HOST_TEST_BIN


if __name__ == "__main__":
    build()
    build_host_test()
    sys.exit(0)
