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


if __name__ == "__main__":
    print(build(verbose=True))
