"""Runs the Python-free check of the C ABI (tests/standalone/rmsnorm_standalone.cpp, the
counterpart of the reference's rmsnorm_standalone.cu) on the GPU.  The executable is built
beforehand on the CPU (`make`, or __graft_entry__.build())."""
import subprocess
from pathlib import Path

import pytest

EXE = Path(__file__).resolve().parent / "standalone" / "rmsnorm_standalone"


@pytest.mark.gpu
def test_standalone_executable_passes():
    if not EXE.exists():
        pytest.fail(f"{EXE} has not been built: run `make` at the repository root")
    out = subprocess.run([str(EXE)], capture_output=True, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "Validation PASSED" in out.stdout
