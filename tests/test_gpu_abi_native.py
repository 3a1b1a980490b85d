"""The C ABI called from a plain C++ program (no Python, no torch in that process)."""
import subprocess
from pathlib import Path

import pytest

PROBE = Path(__file__).resolve().parent / "native" / "abi_probe.bin"


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(256, 384), (200, 72)])
def test_rotate_adam_rotate_from_cpp(rows, cols):
    if not PROBE.exists():
        pytest.fail(f"{PROBE} is not built: run python -m soap_tp_amd.build")
    completed = subprocess.run([str(PROBE), str(rows), str(cols), "3", "1"], capture_output=True, text=True,
                               timeout=100)
    assert completed.returncode == 0, completed.stdout + completed.stderr
    assert completed.stdout.strip().endswith("ok"), completed.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("mode,size", [("qr", 300), ("eigh", 300)])
def test_factorisations_from_cpp_with_library_owned_workspace(mode, size):
    if not PROBE.exists():
        pytest.fail(f"{PROBE} is not built: run python -m soap_tp_amd.build")
    completed = subprocess.run([str(PROBE), mode, str(size)], capture_output=True, text=True, timeout=100)
    assert completed.returncode == 0, completed.stdout + completed.stderr
    assert completed.stdout.strip().endswith("ok"), completed.stdout
