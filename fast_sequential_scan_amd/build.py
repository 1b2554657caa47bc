"""Builds the HIP library for gfx950, in-tree.

    python -m fast_sequential_scan_amd.build

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
The result, ``fast_sequential_scan_amd/_lib/libfss_scan.so``, is a plain C-ABI
shared library (include/fss_scan.h): no torch headers, no pybind.

Translation units (compiled in parallel, then linked):
  csrc/fss_api.hip       the C ABI, planning, small kernels
  csrc/fss_scan_rm.hip   the row-major scan kernels, once per storage type and direction
  csrc/fss_scan_cm.hip   the channel-major scan kernels

``build_torch_binding`` compiles csrc/fss_torch_binding.cpp (host code: the PyTorch-side dispatch of
``scan_cu`` in C++ over that C ABI) into ``_lib/fss_torch_binding.so`` with the host compiler.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from typing import List, Sequence, Tuple

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libfss_scan.so")

# -packed-fp32-ops is switched off on purpose: the packed fp32 forms hipcc would
# otherwise form from scalar float code are not wanted in this library.
HIPCC_FLAGS: List[str] = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]

# (object name, source, extra defines)
UNITS: Sequence[Tuple[str, str, Tuple[str, ...]]] = (
    ("api", "fss_api.hip", ()),
    *(
        (f"rm_{t.lower()}_{name}", "fss_scan_rm.hip",
         (f"-DFSS_RM_ELEM={t}", f"-DFSS_RM_BWD={bwd}", f"-DFSS_RM_LAUNCH=launch_rm_{t.lower()}_{name}"))
        for t in ("BF16", "F16", "F32") for bwd, name in ((0, "fwd"), (1, "bwd"))
    ),
    ("cm", "fss_scan_cm.hip", ()),
)


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise FileNotFoundError("hipcc not found (set HIPCC or install ROCm)")


def _run(cmd: List[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError(f"{os.path.basename(cmd[0])} failed with exit code {proc.returncode}: {' '.join(cmd)}")
    if verbose and proc.stderr and "-Rpass" in " ".join(cmd):
        sys.stderr.write(proc.stderr)


def build(verbose: bool = False, extra_flags: Sequence[str] = (), output: str = LIB_PATH) -> str:
    """Compiles every translation unit (always: nothing is cached) and links `output`."""
    os.makedirs(os.path.dirname(output), exist_ok=True)
    hipcc = hipcc_path()
    with tempfile.TemporaryDirectory(prefix="fss_build_") as tmp:
        objects = [os.path.join(tmp, name + ".o") for name, _src, _defs in UNITS]
        commands = [
            [hipcc, *HIPCC_FLAGS, *extra_flags, *defs, "-c", os.path.join(SRC_DIR, src), "-o", obj]
            for (name, src, defs), obj in zip(UNITS, objects)
        ]
        with ThreadPoolExecutor(max_workers=min(len(commands), os.cpu_count() or 1, 8)) as pool:
            list(pool.map(lambda c: _run(c, verbose), commands))
        linked = output + ".tmp"
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-soname,libfss_scan.so", "-o", linked, *objects], verbose)
        os.replace(linked, output)
    return output


BINDING_NAME = "fss_torch_binding"
BINDING_PATH = os.path.join(LIB_DIR, BINDING_NAME + ".so")


def build_torch_binding(verbose: bool = False, output: str = BINDING_PATH) -> str:
    """Compiles the PyTorch binding (always) against the installed torch's headers and libraries."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    os.makedirs(os.path.dirname(output), exist_ok=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = os.environ.get("CXX") or shutil.which("g++") or "g++"
    includes = [*cpp_extension.include_paths(), os.path.join(rocm, "include"), sysconfig.get_paths()["include"]]
    cmd = [
        cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={BINDING_NAME}",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *(f"-I{path}" for path in includes),
        os.path.join(SRC_DIR, "fss_torch_binding.cpp"), "-o", output + ".tmp",
        # torch is imported before this module is loaded, so its libraries are resolved already
        *(f"-L{path}" for path in cpp_extension.library_paths()),
        "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
    ]
    _run(cmd, verbose)
    os.replace(output + ".tmp", output)
    return output


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_torch_binding(verbose=True))
