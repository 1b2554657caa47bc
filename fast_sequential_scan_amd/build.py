"""Builds the HIP library for gfx950, in-tree.

    python -m fast_sequential_scan_amd.build

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
The result, ``fast_sequential_scan_amd/_lib/libfss_scan.so``, is a plain C-ABI
shared library (include/fss_scan.h): no torch headers, no pybind.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from typing import List

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(PKG_DIR, "csrc", "fss_scan.hip")
LIB_DIR = os.path.join(PKG_DIR, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libfss_scan.so")

# -packed-fp32-ops is switched off on purpose: the packed fp32 forms hipcc would
# otherwise form from scalar float code are not wanted in this library.
HIPCC_FLAGS: List[str] = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise FileNotFoundError("hipcc not found (set HIPCC or install ROCm)")


def build(verbose: bool = False, extra_flags: List[str] = ()) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-o", tmp, SRC]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
