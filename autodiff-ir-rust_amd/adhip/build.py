"""Builds the in-tree shared library `csrc/libadhip.so` with hipcc for gfx950.

The library holds the host side of the device (IR parser, lowering, code generator, runtime); the
device code it launches is generated per program and compiled for gfx950 by hipRTC."""
from __future__ import annotations

import glob
import os
import subprocess

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_PKG_DIR), "csrc")


def build_library(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.cpp")))
    out = os.path.join(CSRC, "libadhip.so")
    cmd = [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
           "-Wno-unused-function", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", out] + srcs + ["-lhiprtc"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return out


def build_cxx_smoke(verbose: bool = False) -> str:
    """Compile tests/cxx/cabi_smoke.cpp (plain C++ against include/adhip.h) and link it with the library."""
    root = os.path.dirname(os.path.dirname(_PKG_DIR))
    src = os.path.join(root, "tests", "cxx", "cabi_smoke.cpp")
    out = os.path.join(root, "tests", "cxx", "cabi_smoke")
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-o", out, src, "-L" + CSRC, "-ladhip", "-Wl,-rpath," + CSRC,
           "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return out


def build_overlap_probe(verbose: bool = False) -> str:
    """Compile tests/cxx/mfma_valu_overlap.cpp (a hardware premise of the matrix kernels, measured) for gfx950."""
    root = os.path.dirname(os.path.dirname(_PKG_DIR))
    src = os.path.join(root, "tests", "cxx", "mfma_valu_overlap.cpp")
    out = os.path.join(root, "tests", "cxx", "mfma_valu_overlap")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-o", out, src]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
