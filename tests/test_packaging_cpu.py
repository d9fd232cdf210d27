"""The build step of the package (setup.py `build_hip`, i.e. mgrrmsnorm_amd._build.build),
run into a scratch directory: hipcc cross-compiles the library for gfx950, g++ builds the torch
extension over it, and both load with the ABI version the Python side expects.  (Reference:
the CUDAExtension recipe, setup.py:23-51.)  No GPU is needed; nothing is launched."""
import ctypes
import importlib.util
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    out = tmp_path_factory.mktemp("mg_build")
    proc = subprocess.run([sys.executable, "setup.py", "build_hip", f"--out-dir={out}"], cwd=ROOT,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    assert proc.returncode == 0, proc.stdout[-4000:]
    return out


def test_build_hip_produces_a_loadable_library(built):
    from mgrrmsnorm_amd import _build, _lib

    lib_path = built / _build.LIB_PATH.name
    assert lib_path.exists()
    lib = ctypes.CDLL(str(lib_path))
    lib.mg_abi_version.restype = ctypes.c_int
    assert lib.mg_abi_version() == _lib.ABI_VERSION
    for name in _lib.SIGNATURES:
        assert hasattr(lib, name), f"{name} missing from the freshly built library"
    # the code object is for gfx950 and nothing else
    blob = lib_path.read_bytes()
    assert b"gfx950" in blob and b"gfx942" not in blob and b"gfx90a" not in blob


def test_build_hip_produces_a_loadable_extension(built):
    from mgrrmsnorm_amd import _build, _lib

    ext_path = built / _build.BINDING_PATH.name
    assert ext_path.exists()
    import torch  # noqa: F401  (the extension links against torch's libraries)

    spec = importlib.util.spec_from_file_location(_build.BINDING_NAME, ext_path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.abi_version() == _lib.ABI_VERSION
    for name in ("rmsnorm_forward", "rmsnorm_backward", "swiglu_forward", "swiglu_backward", "rmsnorm", "swiglu"):
        assert callable(getattr(mod, name))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        mod.rmsnorm_forward(torch.ones(2, 8), torch.ones(8), 1e-6)


def test_package_metadata_lists_what_ships():
    text = (ROOT / "setup.py").read_text()
    for needle in ("libmegagemm_hip.so", "_binding*.so", "megagemm_hip_tuning.h", '"megagemm"', "rmsnorm_cuda_ops"):
        assert needle in text
    assert "csrc/tools" not in text
    manifest = (ROOT / "MANIFEST.in").read_text()
    assert "*.cpp" in manifest and "include/*.h" in manifest
