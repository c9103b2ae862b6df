"""Builds libdejavu_hip.so in-tree with hipcc for gfx950.

Run as ``python -m dejavu_amd.build``; tests and benchmarks only load the
library that this step leaves next to the package.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libdejavu_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 ALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; it is needed to build " + LIB_NAME)
    return exe


def build_library(verbose: bool = True) -> str:
    src = os.path.join(CSRC, "dejavu_hip.hip")
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-I", os.path.join(PKG_DIR, "..", "include"), src, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    print("built", LIB_PATH)
    sys.exit(0)
