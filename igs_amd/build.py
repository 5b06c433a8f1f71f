"""Builds igs_amd/libigs_hip.so (the C-ABI shared library) with hipcc for gfx950.

Usage: python -m igs_amd.build            (from the repository root)
hipcc cross-compiles without a GPU; the built library sits in-tree next to this file.
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
SOURCES = [os.path.join(PKG, "csrc", "igs_gs2d.hip")]
LIB = os.path.join(PKG, "libigs_hip.so")

# Packed-fp32 instruction selection is switched off for all device code.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results land in ordinary VGPRs (the vector ALU reads them without a copy out of
    # the accumulation registers); only the diversity-loss kernel uses the matrix cores
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-I", os.path.join(ROOT, "include"),
]


def build(verbose: bool = True, extra=()) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *extra, "-o", LIB, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def is_stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    csrc = os.path.join(PKG, "csrc")
    deps = [os.path.join(csrc, f) for f in os.listdir(csrc)] + [os.path.join(ROOT, "include", "igs_hip.h")]
    return any(os.path.getmtime(d) > t for d in deps)


if __name__ == "__main__":
    build(extra=sys.argv[1:])
