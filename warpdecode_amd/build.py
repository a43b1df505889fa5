"""Builds libwarpdecode_amd.so (hand-written HIP for gfx950) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libwarpdecode_amd.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",                                   # every rounding is written out in the source
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build(verbose=False):
    cmd = ["hipcc"] + FLAGS + ["-o", LIB, os.path.join(CSRC, "wd_lib.hip")]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return LIB


def build_host_test(verbose=False):
    """The C++ test of the operator header (tests/host/test_wd_ops.cpp): host compiler only, linked against
    the HIP library and the oracle, both found again at run time relative to the binary."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "host", "test_wd_ops.cpp")
    exe = os.path.join(root, "tests", "host", "test_wd_ops")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(root, "include"), "-I" + os.path.join(HERE, "host"),
           "-I" + os.path.join(root, "oracle"), src, "-L" + HERE, "-lwarpdecode_amd", "-L" + os.path.join(root, "oracle"),
           "-lwdoracle", "-Wl,-rpath,$ORIGIN/../../warpdecode_amd", "-Wl,-rpath,$ORIGIN/../../oracle", "-o", exe]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    # the expert prefetcher's host test: no GPU library at all
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-pthread", "-I" + CSRC, os.path.join(root, "tests", "host", "test_prefetch.cpp"),
           "-o", os.path.join(root, "tests", "host", "test_prefetch")]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    # the hand-off word helper of the resident launch: a header of plain C++
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-I" + CSRC, os.path.join(root, "tests", "host", "test_handword.cpp"),
           "-o", os.path.join(root, "tests", "host", "test_handword")]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return exe


if __name__ == "__main__":
    build(verbose=True)
    print("built", LIB)
