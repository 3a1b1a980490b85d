"""Compile the gfx950 kernels into ``soap_tp_amd/libsoap_mi355.so`` with hipcc.

Run as ``python -m soap_tp_amd.build``.  hipcc cross-compiles without a GPU, so this works
on a build host; the resulting shared library is loaded with ctypes by ``soap_tp_amd._native``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / "csrc"
LIBRARY_PATH = PACKAGE_DIR / "libsoap_mi355.so"
INCLUDE_DIR = PACKAGE_DIR.parent / "include"
# A C++ program that calls the C ABI without Python or torch (used by a GPU test and for
# hardware-counter runs, where the profiled program should be a plain executable).
ABI_PROBE_SOURCE = PACKAGE_DIR.parent / "tests" / "native" / "abi_probe.cpp"
ABI_PROBE_PATH = PACKAGE_DIR.parent / "tests" / "native" / "abi_probe.bin"
SOURCES = ("api.hip",)

# -packed-fp32-ops is switched off on purpose: the compiler must not fuse scalar fp32 code
# into v_pk_* instructions on this target.
HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wno-unused-result",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


def hipcc_path() -> str:
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc was not found; the gfx950 kernels cannot be built.")
    return found


def build(verbose: bool = False) -> Path:
    command = [hipcc_path(), *HIPCC_FLAGS]
    command += [str(CSRC_DIR / source) for source in SOURCES]
    command += ["-o", str(LIBRARY_PATH)]
    if verbose:
        print(" ".join(command), flush=True)
    completed = subprocess.run(command, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    stderr = "\n".join(line for line in completed.stderr.splitlines() if noise not in line)
    if completed.returncode != 0:
        raise RuntimeError(f"hipcc failed ({completed.returncode}):\n{stderr}")
    if verbose and stderr.strip():
        print(stderr, file=sys.stderr)
    return LIBRARY_PATH


def build_abi_probe(verbose: bool = False) -> Path:
    """Host-only build of tests/native/abi_probe.cpp against the shared library."""
    command = [hipcc_path(), "-O2", "-std=c++17", "-I", str(INCLUDE_DIR), str(ABI_PROBE_SOURCE),
               "-L", str(PACKAGE_DIR), "-lsoap_mi355", "-Wl,-rpath,$ORIGIN/../../soap_tp_amd",
               "-Wno-unused-result", "-o", str(ABI_PROBE_PATH)]
    if verbose:
        print(" ".join(command), flush=True)
    completed = subprocess.run(command, capture_output=True, text=True)
    if completed.returncode != 0:
        raise RuntimeError(f"hipcc failed ({completed.returncode}):\n{completed.stderr}")
    return ABI_PROBE_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_abi_probe(verbose=True))
