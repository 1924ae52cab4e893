"""Builds the test programs that are compiled code: tests/bin/tl_seam_check, which drives the
backend header cpp-tensorlib_amd/include/tl/hip.h the way the reference's evaluator drives a
backend (tests/seam_check.cpp, plain g++; the GPU tests run it).

    python tests/build_programs.py
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
BIN = os.path.join(HERE, "bin")
SEAM_CHECK = os.path.join(BIN, "tl_seam_check")


def build(verbose=True):
    os.makedirs(BIN, exist_ok=True)
    inc = os.path.join(ROOT, "cpp-tensorlib_amd", "include")
    cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-I", inc, os.path.join(HERE, "seam_check.cpp"),
           "-o", SEAM_CHECK, "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return SEAM_CHECK


if __name__ == "__main__":
    print(build())
